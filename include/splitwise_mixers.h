/*
 * splitwise_mixers.h -- C ABI of libsplitwise_mixers.so (gfx950 / MI355X).
 *
 * Operators of decoders that mix tokens by other means than rotary softmax attention over a full
 * context: recurrent delta-rule layers with a per-sequence state, short causal convolutions,
 * attention over a sliding window plus kept first tokens with the heads' weights mixed after the
 * softmax, norms with a single gain; linear attention with a decay per head, soft-capped gated attention
 * with partial rotary embedding, routed experts with group-limited choice, and the fused residual-add + norm
 * of layers whose sublayers run side by side; attention over chunks with an extra softmax term and over a
 * latent shared by all heads, gated linear attention with a decay per key channel, and the gated residual
 * step of layers that read a mix of all earlier layers' outputs; norms in groups of channels around every
 * sublayer, a causal convolution added to a sublayer's input, the delta rule with one decay per head, attention
 * with sigmoid weights and a softmax router.  A library of its own so that a model that needs only these compiles
 * only these.
 *
 * A step is a RAGGED batch: the new tokens of all sequences back to back in one token dimension.
 *   q_start[B + 1]   first row of every sequence's tokens (int32, ascending, q_start[B] = rows)
 *   ctx_len[B]       tokens of the sequence that earlier steps have run (its first new token's position)
 *   token_seq[rows]  sequence index of every row
 *   state_slot[B]    slot of the sequence in the recurrent-state pools
 *   block_tables[B, table_width]   pages of the sequence in the paged caches
 * A sequence with ctx_len == 0 starts from the empty state whatever its slot holds.
 *
 * Conventions as in splitwise_hip.h: SW_OK / negative status, swm_last_error(), asynchronous
 * launches on `stream`, borrowed tensors.  `act_dtype` is SW_F32 or SW_BF16; everything that the
 * comments call fp32 is fp32 in both.
 */
#ifndef SPLITWISE_MIXERS_H_
#define SPLITWISE_MIXERS_H_

#include <stdint.h>

#include "splitwise_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

#define SWM_ABI_VERSION 5
int swm_abi_version(void);
const char* swm_last_error(void);

/* residual[t] += y[t] / sqrt(mean(y[t]^2) + eps) * gain[0]   (residual fp32, y of y_dtype, gain fp32)
 * and, when `cast_out` is not NULL, cast_out[t] = act_dtype(residual[t]). */
int swm_scalar_norm_add(float* residual, const void* y, const float* gain, float eps, void* cast_out,
                        int64_t rows, int width, int64_t y_stride, int y_dtype, int act_dtype, void* stream);
/* out[t] = act_dtype(x[t] / sqrt(mean(x[t]^2) + eps) * gain[0]), x fp32. */
int swm_scalar_norm(void* out, const float* x, const float* gain, float eps, int64_t rows, int width,
                    int act_dtype, void* stream);

/* Query / key norm over the WHOLE projection and the cache write of one attention layer.
 * q_out[t] (fp32, [rows, q_size]) = q[t] / sqrt(mean(q[t]^2) + eps) * q_gain.  With k != NULL:
 * key_cache[slot] = k[t] / sqrt(mean(k[t]^2) + eps) * k_gain and value_cache[slot] = v[t], where
 * slot = slot_mapping[t] (int64, < 0: row not cached); caches are [slots, k_size] / [slots, v_size]
 * in act_dtype. */
int swm_qk_norm_cache(float* q_out, const void* q, const void* k, const void* v, int64_t in_stride,
                      const float* q_gain, const float* k_gain, float eps, void* key_cache, void* value_cache,
                      const int64_t* slot_mapping, int64_t rows, int q_size, int k_size, int v_size,
                      int act_dtype, void* stream);

/* Attention of every new token over its sequence's paged keys: position i sees j <= i with
 * i - j < window or j < keep_first; softmax over those; then head h's weights become
 * sum_g talk[h, g] * weights_g and are applied to the values of h's own key/value head.
 * q fp32 [rows, heads * dim]; caches [pages * page_size, kv_heads * dim | vdim] act_dtype;
 * talk fp32 [heads, heads]; out act_dtype [rows, heads * vdim].
 * `splits` > 1 (steps of few tokens): every token's visible keys are cut into that many runs, one workgroup
 * each, joined by a second launch; `partial` then holds rows * splits * (2 * heads + heads * kv_heads * vdim)
 * floats of scratch. */
int swm_window_attention(void* out, const float* q, const void* key_cache, const void* value_cache,
                         const float* talk, const int32_t* block_tables, int table_width,
                         const int32_t* q_start, const int32_t* ctx_len, const int32_t* token_seq,
                         int64_t rows, int num_seqs, int heads, int kv_heads, int dim, int vdim, int page_size,
                         float scale, int window, int keep_first, int splits, float* partial, int act_dtype,
                         void* stream);

/* Short causal convolution over time per channel, then silu.  x act_dtype [rows, channels] (row stride
 * x_stride); taps fp32 [channels, num_taps], last column = current token; state fp32
 * [slots, num_taps - 1, channels] = the sequence's last num_taps - 1 inputs; out fp32 [rows, channels].
 * swm_short_conv reads the state; swm_short_conv_advance then moves it past the step's tokens. */
int swm_short_conv(float* out, const void* x, int64_t x_stride, const float* taps, const float* state,
                   const int32_t* q_start, const int32_t* ctx_len, const int32_t* token_seq,
                   const int32_t* state_slot, int64_t rows, int channels, int num_taps, int act_dtype,
                   void* stream);
int swm_short_conv_advance(float* state, const void* x, int64_t x_stride, const int32_t* q_start,
                           const int32_t* ctx_len, const int32_t* state_slot, int num_seqs, int channels,
                           int num_taps, int act_dtype, void* stream);

/* Delta rule with a gate and a decay per head and key channel, token by token per sequence:
 *   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
 * with q, k made unit vectors per head (eps 1e-6 inside the root; q also times dim^-1/2),
 * beta = sigmoid(beta_pre), g = exp(-exp(a_log[head]) * softplus(decay_pre + dt_bias)).
 * qkv fp32 [rows, 2 * kv_heads * dim + heads * vdim] (q | k | v after the short convolution);
 * beta_pre act_dtype [rows, heads] (row stride beta_stride); decay_pre act_dtype [rows, heads * dim];
 * dt_bias fp32 [heads * dim]; a_log fp32 [heads]; state fp32 [slots, heads, dim, vdim];
 * out fp32 [rows, heads * vdim].  `workspace`: swm_channel_delta_workspace_floats() floats for the operands that
 * a prologue kernel, parallel over tokens, prepares for the recurrence. */
int64_t swm_channel_delta_workspace_floats(int64_t rows, int heads, int dim);
int swm_channel_delta(float* out, const float* qkv, const void* beta_pre, int64_t beta_stride,
                      const void* decay_pre, const float* dt_bias, const float* a_log, float* state,
                      const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot, int64_t rows,
                      int num_seqs, int heads, int kv_heads, int dim, int vdim, float* workspace, int act_dtype,
                      void* stream);

/* Delta rule with a decay and a removal rate per head and key channel:
 *   S <- diag(w) S - (a * u) (u^T S) + k v^T   (both terms read the old S);  o = S^T r
 * u = k / sqrt(sum k^2 + 1e-6), w = exp(-exp(-1/2) sigmoid(decay_pre + w0)), a = sigmoid(rate_pre + a_bias).
 * r, k, v act_dtype [rows, heads * dim] (row stride rkv_stride); decay_pre, rate_pre act_dtype
 * [rows, heads * dim] (row strides given); w0, a_bias fp32 [heads * dim]; state fp32 [slots, heads, dim, dim];
 * out fp32 [rows, heads * dim]. */
int swm_general_delta(float* out, const void* r, const void* k, const void* v, int64_t rkv_stride,
                      const void* decay_pre, int64_t decay_stride, const float* w0, const void* rate_pre,
                      int64_t rate_stride, const float* a_bias, float* state, const int32_t* q_start,
                      const int32_t* ctx_len, const int32_t* state_slot, int64_t rows, int num_seqs, int heads,
                      int dim, float* workspace, int act_dtype, void* stream);
int64_t swm_general_delta_workspace_floats(int64_t rows, int heads, int dim);

/* out[t, h, :] = act_dtype(o / sqrt(mean(o^2) + eps) * weight[h * weight_head_stride + :] * sigmoid(gate[t, h, :]))
 * o fp32 [rows, heads * vdim]; gate act_dtype (row stride gate_stride); weight fp32. */
int swm_head_norm_gate(void* out, const float* o, const void* gate, int64_t gate_stride, const float* weight,
                       int weight_head_stride, float eps, int64_t rows, int heads, int vdim, int act_dtype,
                       void* stream);

/* Feed-forward experts over (row, choice) pairs sorted by expert: `order` (int32 [pairs]) holds
 * row * top + choice of every sorted pair and expert e owns the sorted pairs
 * [expert_start[e], expert_start[e + 1]).
 * hidden[pair] = gelu_erf(up[e] x[order[pair] / top])   (act_dtype [pairs, ff]; up act_dtype [experts, ff, width]) */
int swm_expert_up_gelu(void* hidden, const void* x, const void* up, const int32_t* order,
                       const int32_t* expert_start, int num_experts, int64_t sorted_rows, int width, int ff,
                       int top, int act_dtype, void* stream);
/* out[order[pair] / top] += weight * down[e] hidden[pair]   (out fp32 [rows, width], zeroed by the caller;
 * down act_dtype [experts, width, ff]; atomic adds when top > 1). */
int swm_expert_down(float* out, const void* hidden, const void* down, const int32_t* order,
                    const int32_t* expert_start, int num_experts, int64_t sorted_rows, int width, int ff,
                    int top, float weight, int act_dtype, void* stream);

/* The same two steps with the hidden layer's activation named (SWM_ACT_GELU: exact gelu, SWM_ACT_RELU2: the square
 * of relu) and with a weight per (row, choice) pair: out[row] += weight * pair_weight[row * top + choice] * ...
 * (pair_weight fp32 [rows * top], NULL: all 1). */
#define SWM_ACT_GELU 0
#define SWM_ACT_RELU2 1
#define SWM_ACT_NONE 2 /* the products as they are: the hidden layer's gated unit is a kernel of its own */
#define SWM_ACT_CLAMPED_GLU 3 /* swm_expert_up_as only: a gated hidden layer with limits in the kernel's epilogue */
int swm_expert_up(void* hidden, const void* x, const void* up, const int32_t* order, const int32_t* expert_start,
                  int num_experts, int64_t sorted_rows, int width, int ff, int top, int activation, int act_dtype,
                  void* stream);
/* swm_expert_up with the gated unit of swm_clamped_glu in its epilogue (activation SWM_ACT_CLAMPED_GLU; the other
 * activations ignore the three numbers): `up` then holds 32 * ceil(ff / 16) rows per expert -- per run of 16 hidden
 * channels its 16 gate rows followed by its 16 up rows, a shorter last run padded with zero rows -- and
 * hidden[pair, c] = g sigmoid(glu_alpha g) (u + glu_shift), g = min(gate x, glu_limit), u = clamp(up x, +-glu_limit). */
int swm_expert_up_as(void* hidden, const void* x, const void* up, const int32_t* order, const int32_t* expert_start,
                     int num_experts, int64_t sorted_rows, int width, int ff, int top, int activation, float glu_alpha,
                     float glu_limit, float glu_shift, int act_dtype, void* stream);
int swm_expert_down_weighted(float* out, const void* hidden, const void* down, const int32_t* order,
                             const int32_t* expert_start, int num_experts, int64_t sorted_rows, int width, int ff,
                             int top, float weight, const float* pair_weight, int act_dtype, void* stream);

/* ---- layers whose two sublayers read one norm of an fp32 residual stream ---- */

/* residual[t] += a[t] + b[t] + c[t] (each may be NULL; a, b act_dtype with row strides, c fp32 contiguous; the
 * addends are summed first), then, when `out` is not NULL,
 * out[t] = act_dtype(residual[t] / sqrt(mean(residual[t]^2) + eps) * (offset + weight)), weight fp32 [width]. */
int swm_stream_add_norm(float* residual, const void* a, int64_t a_stride, const void* b, int64_t b_stride,
                        const float* c, const float* weight, float offset, float eps, void* out, int64_t rows,
                        int width, int act_dtype, void* stream);

/* in [rows, 2 * ff] = gate | up (row stride in_stride):  g = min(gate, limit), u = clamp(up, -limit, limit),
 * out[rows, ff] = g * sigmoid(alpha * g) * (u + shift).  limit may be +inf. */
int swm_clamped_glu(void* out, const void* in, int64_t in_stride, int64_t rows, int ff, float alpha, float limit,
                    float shift, int act_dtype, void* stream);
/* out[rows, ff] = max(in, 0)^2 */
int swm_relu2(void* out, const void* in, int64_t in_stride, int64_t rows, int ff, int act_dtype, void* stream);

/* Rotary embedding on the first rot_dims coordinates of every head: pair i is the neighbours (2i, 2i + 1), or with
 * pair_halves != 0 the coordinates (i, i + rot_dims / 2); angle
 * = float(positions[t]) * inv_freq[i] in fp32 (inv_freq fp32 [rot_dims / 2]); the other coordinates pass.
 * q_out fp32 [rows, heads * dim] = rotated q.  With k != NULL: key_cache[slot] = rotated k, value_cache[slot] = v
 * (slot = slot_mapping[t], < 0: not cached; caches [slots, kv_heads * dim | vdim] act_dtype).  q, k, v are column
 * ranges of one projection output (row stride in_stride). */
int swm_rope_cache(float* q_out, const void* q, const void* k, const void* v, int64_t in_stride,
                   const int64_t* positions, const float* inv_freq, int rot_dims, int pair_halves, void* key_cache,
                   void* value_cache, const int64_t* slot_mapping, int64_t rows, int heads, int kv_heads, int dim,
                   int vdim, int act_dtype, void* stream);

/* The choice of a mixture-of-experts router from its logits (fp32 [rows, experts], the router's product with the
 * layer input): s = sigmoid(logit); choice scores s + correction (NULL: none); experts form `groups` equal groups
 * of neighbours, a group scores the sum of its two largest choice scores and only the best `keep` groups stay in the
 * choice (groups == 1 or keep == groups: all); the `top` largest choice scores are chosen; weights = s of the chosen
 * / (their sum + 1e-20) * scale.  chosen int32 [rows, top], weights fp32 [rows, top]. */
int swm_group_router(int32_t* chosen, float* weights, const float* logits, const float* correction, int64_t rows,
                     int experts, int top, int groups, int keep, float scale, void* stream);

/* chosen (int32 [pairs], every value in [0, experts)) -> order (int32 [pairs]: the pair indices grouped by expert) and
 * expert_start (int32 [experts + 1]: every expert's first place in `order`); what the expert kernels take. */
int swm_group_pairs(int32_t* order, int32_t* expert_start, const int32_t* chosen, int64_t pairs, int experts,
                    void* stream);

/* Causal softmax attention of every new token over its sequence's paged keys with grouped query heads (query head
 * h reads key/value head h / (heads / kv_heads)): score = (q . k) * scale, then softcap * tanh(score / softcap) when
 * softcap > 0; position i sees j <= i (and i - j < window when window > 0); fp32 scores, weights and sums.
 * q fp32 [rows, heads * dim] (already rotated); caches [pages * page_size, kv_heads * dim | vdim] act_dtype;
 * gate (NULL: none) act_dtype [rows, heads * vdim] with row stride: the output is multiplied by sigmoid(gate);
 * out act_dtype [rows, heads * vdim].  max_query_len: the most new tokens of any sequence (0: unknown); steps of
 * few tokens per sequence split every sequence's keys over the waves of a workgroup. */
int swm_capped_attention(void* out, const float* q, const void* key_cache, const void* value_cache,
                         const void* gate, int64_t gate_stride, const int32_t* block_tables, int table_width,
                         const int32_t* q_start, const int32_t* ctx_len, int64_t rows, int num_seqs,
                         int max_query_len, int heads, int kv_heads, int dim, int vdim, int page_size, float scale,
                         float softcap, int window, int act_dtype, void* stream);

/* The same attention with the mask and the cache layout named: `window` > 0: position i sees j with 0 <= i - j <
 * window; `chunk` > 0: i sees j <= i with j / chunk == i / chunk (chunks count from position 0 of the sequence); both
 * 0: every j <= i.  `sink` != 0: the softmax's denominator has one more term, exp(0) (a key of score 0 without a
 * value).  A cache slot (one token) holds k_stride / v_stride elements, of which key/value head g's begin at g * dim /
 * g * vdim: value_cache may point into the key cache (values that are a part of the key row).  Key and value sizes up
 * to 512.  Steps of few rows per sequence and few sequences share a tile's keys out among several workgroups, joined
 * by a second launch: `workspace` then holds swm_masked_attention_workspace_floats() floats (0: not such a step;
 * NULL: never shared out). */
int64_t swm_masked_attention_workspace_floats(int64_t rows, int num_seqs, int max_query_len, int heads, int kv_heads,
                                              int vdim, int page_size, int table_width, int window, int chunk);
int swm_masked_attention(void* out, const float* q, const void* key_cache, const void* value_cache, const void* gate,
                         int64_t gate_stride, const int32_t* block_tables, int table_width, const int32_t* q_start,
                         const int32_t* ctx_len, int64_t rows, int num_seqs, int max_query_len, int heads,
                         int kv_heads, int dim, int vdim, int page_size, float scale, float softcap, int window,
                         int chunk, int sink, int64_t k_stride, int64_t v_stride, float* workspace, int act_dtype,
                         void* stream);

/* ---- layers whose sublayer outputs enter an fp32 stream through a gate, with a mix over all earlier layers ---- */

/* v = stream[t] + mult * y[t] * sigmoid(gate[t])   (y NULL: v = stream[t]; gate NULL: no gate; y, gate act_dtype
 * with row strides).  With `history` (fp32 [entries or more, rows, width], layer_stride floats apart): entry
 * entries - 1 receives v, and v becomes sum_j depth_weights[j] * history[j] over the `entries` entries (fp32 weights).
 * stream[t] = v.  With `out`: out[t] = act_dtype(tanh(norm_alpha[0] * v) * norm_weight + norm_bias), all fp32. */
int swm_gated_stream_step(float* stream, const void* y, int64_t y_stride, const void* gate, int64_t gate_stride,
                          float mult, float* history, int64_t layer_stride, const float* depth_weights, int entries,
                          const float* norm_alpha, const float* norm_weight, const float* norm_bias, void* out,
                          int64_t rows, int width, int act_dtype, void* stream_handle);

/* out[t] = c0 U(z) + c1 U(z^2) + c2 U(z^3) + c3, powers element by element, U(u) = u / sqrt(mean(u^2) + eps) over the
 * row's ff values; coef fp32 [4]; z act_dtype with row stride; out act_dtype [rows, ff]. */
int swm_poly_norm(void* out, const void* z, int64_t z_stride, const float* coef, float eps, int64_t rows, int ff,
                  int act_dtype, void* stream);

/* out[t, h * size + c] = y[t, h, c] * sigmoid(gate[t, h * size + c])   (silu != 0: * gate * sigmoid(gate));
 * y addressed as t * y_row_stride + h * y_head_stride + c. */
int swm_gate_mul(void* out, const void* y, int64_t y_row_stride, int64_t y_head_stride, const void* gate,
                 int64_t gate_stride, int64_t rows, int heads, int size, int silu, int act_dtype, void* stream);

/* Attention over a low-rank latent: a token's cache row is its latent (rank) | one rotated key part (rot) shared by
 * all heads.  cache[slot] = down[t, :rank] / sqrt(mean(.^2) + eps) * norm_weight | rotate(down[t, rank:rank + rot])
 * (down NULL: no cache write); q_out[t, h] (fp32 [rows, heads * (rank + rot)]) = q_latent[t, h] | rotate(q_rot[t, h]),
 * q_latent being the head's query already taken through the key up-projection.  Rotation on neighbouring pairs,
 * angle = float(position) * inv_freq[i] (fp32 [rot / 2]).  q_latent, q_rot are addressed by row and head strides. */
int swm_latent_rope_cache(float* q_out, const void* q_latent, int64_t ql_row_stride, int64_t ql_head_stride,
                          const void* q_rot, int64_t qr_row_stride, int64_t qr_head_stride, const void* down,
                          int64_t down_stride, const float* norm_weight, float eps, const int64_t* positions,
                          const float* inv_freq, void* cache, const int64_t* slot_mapping, int64_t rows, int heads,
                          int rank, int rot, int act_dtype, void* stream);

/* The per-head output norm with the gate's activation named: gate_silu != 0 multiplies by gate * sigmoid(gate). */
int swm_head_norm_gate_act(void* out, const float* o, const void* gate, int64_t gate_stride, const float* weight,
                           int weight_head_stride, float eps, int64_t rows, int heads, int vdim, int gate_silu,
                           int act_dtype, void* stream);

/* Gated linear attention with a decay per head and key channel:  S <- diag(a_t) S + k_t v_t^T;  o_t = S^T q_t * q_scale,
 * a_t = sigmoid(decay_pre + decay_bias)^(1 / tau), i.e. log a_t = logsigmoid(.) / tau, worked out in fp32.
 * q, k [rows, heads * dim], v [rows, heads * vdim]: act_dtype column ranges of one projection output (row stride
 * in_stride); decay_pre act_dtype [rows, heads * dim] (row stride decay_stride); decay_bias fp32 [heads * dim] (NULL:
 * none); state fp32 [slots, heads, dim, vdim]; out fp32 [rows, heads * vdim].  Key size up to 256.
 * max_query_len: the most new tokens of any sequence (0: unknown).  Long runs are cut into segments that run side by
 * side and are joined by a scan over their end states; `workspace` then holds swm_gla_workspace_floats() floats (0:
 * the step has no long run; NULL: never cut). */
int64_t swm_gla_workspace_floats(int64_t rows, int num_seqs, int max_query_len, int heads, int dim, int vdim);
int swm_gla(float* out, const void* q, const void* k, const void* v, int64_t in_stride, const void* decay_pre,
            int64_t decay_stride, const float* decay_bias, float tau, float q_scale, float* state,
            const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot, int64_t rows, int num_seqs,
            int max_query_len, int heads, int dim, int vdim, float* workspace, int act_dtype, void* stream);

/* Linear attention with one decay per head:  S <- decay[h] S + k v^T;  o = S^T q, with q, k, v = silu of the given
 * projections (act_dtype, column ranges of one output with row stride in_stride; q, k [rows, heads * dim],
 * v [rows, heads * vdim]); decay fp32 [heads]; state fp32 [slots, heads, dim, vdim]; out fp32 [rows, heads * vdim].
 * max_query_len: the most new tokens of any sequence (0: unknown).  Long runs are cut into segments that run side by
 * side and are joined by a scan over their end states; `workspace` then holds swm_lightning_workspace_floats() floats
 * (0: the step has no long run; NULL: never cut). */
int64_t swm_lightning_workspace_floats(int64_t rows, int num_seqs, int max_query_len, int heads, int dim, int vdim);
int swm_lightning(float* out, const void* q, const void* k, const void* v, int64_t in_stride, const float* decay,
                  float* state, const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot, int64_t rows,
                  int num_seqs, int max_query_len, int heads, int dim, int vdim, float* workspace, int act_dtype,
                  void* stream);

/* ---- layers with a norm before AND after each sublayer, taken in groups of channels ---- */

/* N(u; w): the row cut into `groups` equal runs of channels, each run divided by its own sqrt(mean(run^2) + eps),
 * the row times w (fp32 [width]).  With y1:  residual[t] += layer_scale * N(s1 * y1[t] + s2 * y2[t]; post_w)
 * (y2 NULL: one addend; layer_scale fp32 [width] or NULL; y1, y2 of y_dtype with row strides).  With out:
 * out[t] = out_dtype(N(residual[t]; w)) of the new residual.  residual fp32 [rows, width]. */
int swm_group_norm_add(float* residual, const void* y1, int64_t y1_stride, float s1, const void* y2,
                       int64_t y2_stride, float s2, int y_dtype, const float* post_w, const float* layer_scale,
                       const float* w, void* out, int out_dtype, int groups, float eps, int64_t rows, int width,
                       void* stream);

/* The short causal convolution of swm_short_conv with the types and the form named: x of x_dtype, out of out_dtype
 * [rows, channels]; out = act(conv(x) + (residual != 0 ? x : 0)), act = silu when silu != 0.  The state holds the last
 * num_taps - 1 inputs in fp32; advance != 0: the same launch moves it past the step's tokens (else
 * swm_short_conv_advance with x's dtype does). */
int swm_causal_conv(void* out, int out_dtype, const void* x, int x_dtype, int64_t x_stride, const float* taps,
                    float* state, const int32_t* q_start, const int32_t* ctx_len, const int32_t* token_seq,
                    const int32_t* state_slot, int64_t rows, int channels, int num_taps, int silu, int residual,
                    int advance, void* stream);

/* swm_channel_delta with ONE decay per head: g = exp(-exp(a_log[head]) * softplus(decay_pre[t, head] + dt_bias[head])),
 * decay_pre act_dtype [rows, heads] (row stride decay_stride), dt_bias fp32 [heads].  Workspace as swm_channel_delta. */
int swm_gated_delta(float* out, const float* qkv, const void* beta_pre, int64_t beta_stride, const void* decay_pre,
                    int64_t decay_stride, const float* dt_bias, const float* a_log, float* state,
                    const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot, int64_t rows,
                    int num_seqs, int heads, int kv_heads, int dim, int vdim, float* workspace, int act_dtype,
                    void* stream);

/* The same rule in chunks of 32 tokens on the matrix cores, for steps that bring long runs (any step is right, steps of
 * few tokens per sequence are faster with swm_gated_delta): a prologue parallel over (chunk, head), then one walk over
 * each sequence's chunks.  Key sizes up to 224.  `workspace`: swm_gated_delta_chunked_workspace_floats() floats. */
int64_t swm_gated_delta_chunked_workspace_floats(int64_t rows, int num_seqs, int heads, int dim, int vdim);
int swm_gated_delta_chunked(float* out, const float* qkv, const void* beta_pre, int64_t beta_stride,
                            const void* decay_pre, int64_t decay_stride, const float* dt_bias, const float* a_log,
                            float* state, const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot,
                            int64_t rows, int num_seqs, int heads, int kv_heads, int dim, int vdim, float* workspace,
                            int act_dtype, void* stream);

/* swm_rope_cache behind an RMS norm of every query and key head over its `dim` coordinates:
 * x / sqrt(mean(x^2) + norm_eps) * q_norm (k_norm), fp32 [dim] weights shared by the heads; q_norm NULL: no norm. */
int swm_norm_rope_cache(float* q_out, const void* q, const void* k, const void* v, int64_t in_stride,
                        const float* q_norm, const float* k_norm, float norm_eps, const int64_t* positions,
                        const float* inv_freq, int rot_dims, int pair_halves, void* key_cache, void* value_cache,
                        const int64_t* slot_mapping, int64_t rows, int heads, int kv_heads, int dim, int vdim,
                        int act_dtype, void* stream);

/* Attention WITHOUT a softmax over the layout of swm_masked_attention: a key that position i sees (j <= i, and
 * i - j < window when window > 0) weighs sigmoid((q . k) * scale + score_bias[head]) (score_bias fp32 [heads]); the
 * weights are not normalised over the keys.  Gate, caches, workspace (swm_masked_attention_workspace_floats) as there. */
int swm_sigmoid_attention(void* out, const float* q, const void* key_cache, const void* value_cache, const void* gate,
                          int64_t gate_stride, const float* score_bias, const int32_t* block_tables, int table_width,
                          const int32_t* q_start, const int32_t* ctx_len, int64_t rows, int num_seqs,
                          int max_query_len, int heads, int kv_heads, int dim, int vdim, int page_size, float scale,
                          int window, float* workspace, int act_dtype, void* stream);

/* swm_group_router with the scores, the groups' scores and the weights named: softmax != 0: s = softmax(logits) over
 * all experts (else sigmoid); group_best_one != 0: a group scores its largest choice score (else the sum of its two
 * largest); normalize == 0: weights = s of the chosen * scale, not divided by their sum. */
int swm_group_router_as(int32_t* chosen, float* weights, const float* logits, const float* correction, int64_t rows,
                        int experts, int top, int groups, int keep, float scale, int softmax, int group_best_one,
                        int normalize, void* stream);

#ifdef __cplusplus
}
#endif
#endif
