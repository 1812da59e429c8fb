/*
 * lv_mixers.h — C ABI of liblvmix.so: the MI355X (gfx950) kernels of the sequence mixers and the
 * residual machinery that are not plain softmax attention over a full causal context:
 *
 *   lv_hc_update_norm        hyper-connection stream update fused with the next sublayer's stream
 *                            read-out and grouped RMS norm
 *   lv_residual_add_norm     single f32 residual: adds up to two sublayer outputs, RMS norm with weight (offset + w)
 *   lv_clamped_glu           clamped gated linear unit  min(g, L) * sigmoid(alpha g) * (clamp(u, -L, L) + 1)
 *   lv_delta_prep            short causal convolution + silu over the q/k/v channels of a ragged step,
 *                            unit-norm q and k, write strength and decay of the gated delta rule
 *   lv_conv_state_update     carries the last taps-1 convolution inputs of every sequence
 *   lv_gated_delta_rule      the recurrence itself, state in 32-bit, any number of new tokens per sequence
 *   lv_head_norm_gate        per-head RMS norm of the read-out times weight times silu(gate)
 *   lv_qk_fullnorm_store     RMS norm over the whole q and k projection, K/V scatter into the paged cache
 *   lv_pool_update           means of completed blocks of P cached keys and values
 *   lv_window_pool_attn      sliding-window attention over cached tokens plus pooled blocks that lie
 *                            before the window, softmax with an optional zero-score sink, sigmoid output gate;
 *                            with a window no sequence reaches, no pool and no sink it is plain causal attention,
 *                            and with row strides of their own K and V may be views of one wider cache row
 *   lv_latent_prep           latent attention: RMS norm of the query latent, RMS norm of the key/value latent and
 *                            rotation of the shared positional key part, both written into the paged latent cache
 *   lv_latent_q_finish       joins the absorbed queries with their rotated positional part
 *   lv_latent_out_gate       per-head outputs [H, T, Dv] -> [T, H*Dv] times sigmoid(gate), gate per head or per channel
 *   lv_moe_route             sigmoid router with a selection-only correction, group limit and top-k
 *   lv_router_logits         f32 router logits of steps of few tokens, straight from the activations
 *   lv_relu2_scale           squared relu of the experts' up projections times the routing weight
 *   lv_moe_grouped_ff        the experts' feed-forward on rows sorted by expert (grouped GEMMs on the matrix cores)
 *   lv_moe_sort, lv_moe_combine   its first and last step alone, for callers that multiply the sorted rows themselves
 *   lv_sandwich_add_norm     single f32 residual of layers that norm both sides of a sublayer: adds the RMS-normed
 *                            sublayer output, a row of activations and a vector, RMS norm with weight (offset + w)
 *   lv_rotary_store          rotation of part of every query and key head, a factor per query head, K/V scatter
 *                            into the paged cache
 *   lv_polynorm              c1 R(z) + c2 R(z^2) + c3 R(z^3) + c0 with R the division by a row's root mean square
 *   lv_expert_glu            clamped gated unit of several experts side by side with a factor per (token, expert)
 *                            on the pre-activations and a sigmoid per token on the result
 *   lv_moe_grouped_glu_ff    the gathered feed-forward for clamped gated experts whose routing weight scales the
 *                            expert's input
 *   lv_residual_dyt          single f32 residual: adds a sublayer output, or the scaled sum of two RMS-normed and weighted
 *                            ones (two mixers side by side), then the dynamic-tanh norm tanh(alpha x) w + b
 *   lv_qk_prep_store         lv_rotary_store with the pairing of rotated entries as a choice and an optional division of
 *                            every query and key head by its root mean square
 *   lv_masked_attn(_mfma)    lv_window_pool_attn(_mfma) with kept first tokens, chunked visibility and a learned sink per head
 *   lv_lightning_attn        linear attention with a constant decay per head: S <- d S + k v^T, o = S^T q, state in f32
 *   lv_glu_act               act(gate) * up
 *   lv_moe_route_scored      lv_moe_route with softmax scores and groups ranked by their best expert as choices
 *   lv_expert_act_scale      lv_relu2_scale with the activation as a choice
 *   lv_moe_grouped_act_ff    lv_moe_grouped_ff with the activation as a choice and experts that hand their input through
 *   lv_scaled_row_add        y[t] += (sum of a token's factors) * h[t]
 *
 * A "ragged step" is a batch of B sequences; sequence b brings cu_q[b+1]-cu_q[b] new tokens that
 * follow ctx_lens[b] tokens already in the cache / state (a whole prompt, a portion of one, or one
 * decoded token: the kernels make no difference). tok_seq[t] is the sequence of packed token t.
 *
 * Conventions: device pointers; `dtype` LV_MIX_BF16 or LV_MIX_F32 is the element type of activations,
 * caches and convolution state ("act"); vectors named *_w, the stream tensor, recurrent state and
 * everything documented as f32 are 32-bit floats; index tensors int32; strides in elements; every
 * call only enqueues on `stream` (void* hipStream_t), allocates nothing and never synchronises.
 * Return 0 or a negative code; lv_mix_last_error() gives the message.
 */
#ifndef LV_MIXERS_H
#define LV_MIXERS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LV_MIX_ABI_VERSION 7
#define LV_MIX_BF16 0
#define LV_MIX_F32 1
#define LV_MIX_MAX_STREAMS 8
#define LV_MIX_GATE_SILU 0
#define LV_MIX_GATE_SIGMOID 1
#define LV_MIX_GATE_PER_HEAD 0
#define LV_MIX_GATE_PER_CHANNEL 1
#define LV_MIX_ACT_RELU2 0        /* relu(z)^2 */
#define LV_MIX_ACT_GELU_ERF 1     /* z Phi(z), exact */
#define LV_MIX_ACT_GELU_TANH 2    /* 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))) */
#define LV_MIX_SCORE_SIGMOID 0
#define LV_MIX_SCORE_SOFTMAX 1
#define LV_MIX_GROUP_TOP2_SUM 0   /* a group of experts is ranked by the sum of its two highest selection scores */
#define LV_MIX_GROUP_MAX 1        /* ... by its highest */

int lv_mix_abi_version(void);
const char* lv_mix_last_error(void);

/* x [T, S, W] f32, updated in place when y != NULL:  x'[t'] = sum_s mix[s, t'] x[s] + out_w[t'] * y.
 * When out != NULL:  u = sum_s in_w[s] x'[s];  out = grouped_rms_norm(u) * norm_w  (groups equal
 * consecutive parts, each divided by its own sqrt(mean(part^2) + eps)).  y, out: act [T, W]. */
int lv_hc_update_norm(void* x, const void* y, const void* mix, const void* out_w, const void* in_w,
                      const void* norm_w, void* out, int64_t T, int S, int W, int groups, float eps,
                      int dtype, void* stream);

/* x f32 [T, W] += y1 + y2 (act [T, W], either may be NULL), in place; when out != NULL:
 * out act [T, W] = x / sqrt(mean(x^2) + eps) * (w_offset + w), w f32 [W]. */
int lv_residual_add_norm(void* x, const void* y1, const void* y2, const void* w, float w_offset, void* out, int64_t T,
                         int W, float eps, int dtype, void* stream);

/* in act [T, 2F] (row stride ld_in) = [gate | up];  out act [T, F]. */
int lv_clamped_glu(const void* in, int64_t ld_in, void* out, int64_t T, int F, float limit, float alpha,
                   int dtype, void* stream);

/* proj act [T, ld]: columns [0, G*D) q, [G*D, 2*G*D) k, [2*G*D, 2*G*D + H*Dv) v (the convolution
 * channels, C of them), b at column off_b (H wide). a act, rows of stride ld_a: the decay inputs, H numbers, or with
 * decay_per_channel H*D (one for each key channel of each head; dt_bias is as wide as a row of a, A_log always [H]).
 * conv_w f32 [C, taps] (last column = current token); conv_state act [slots, taps-1, C].
 * Outputs f32: qn [T, G, D] (unit norm times D^-1/2), kn [T, G, D], v [T, H, Dv], beta [T, H],
 * decay [T, H] or [T, H, D] = exp(-exp(A_log) * softplus(a + dt_bias)). */
int lv_delta_prep(const void* proj, int64_t ld, const void* conv_w, const void* conv_state,
                  const void* A_log, const void* dt_bias, const int32_t* cu_q, const int32_t* ctx_lens,
                  const int32_t* slots, const int32_t* tok_seq, void* qn, void* kn, void* v, void* beta,
                  void* decay, int64_t T, int G, int H, int D, int Dv, int taps, int off_b, const void* a,
                  int64_t ld_a, int decay_per_channel, float unit_eps, int dtype, void* stream);

int lv_conv_state_update(const void* proj, int64_t ld, void* conv_state, const int32_t* cu_q,
                         const int32_t* ctx_lens, const int32_t* slots, int B, int C, int taps, int dtype,
                         void* stream);

/* state f32 [slots, H, D, Dv], read unless ctx_lens[b] == 0, written back.  o f32 [T, H, Dv].
 * decay f32 [T, H], or [T, H, D] with decay_per_channel: row d of a head's state is multiplied by its own number. */
int lv_gated_delta_rule(const void* qn, const void* kn, const void* v, const void* beta, const void* decay,
                        void* state, const int32_t* cu_q, const int32_t* ctx_lens, const int32_t* slots,
                        void* o, int B, int G, int H, int D, int Dv, int decay_per_channel, void* stream);

/* out act [T, H*Dv] = o / sqrt(mean_dv(o^2) + eps) * norm_w[dv] * act(gate), act = silu or sigmoid (LV_MIX_GATE_*);
 * gate act rows of stride ld_gate. */
int lv_head_norm_gate(const void* o, const void* gate, int64_t ld_gate, const void* norm_w, void* out,
                      int64_t T, int H, int Dv, float eps, int gate_act, int dtype, void* stream);

/* q act [T, H*D] (row stride ld), k [T, G*D], v [T, G*Dv] rows of the same stride.  q_out act [T, H*D]
 * contiguous = rms_norm(q over all H*D) * q_w; k likewise into k_cache [pages, page, G, D]; v copied into
 * v_cache [pages, page, G, Dv] at the slot of position ctx_lens[b] + index in the step. */
int lv_qk_fullnorm_store(const void* q, const void* k, const void* v, int64_t ld, const void* q_w,
                         const void* k_w, void* q_out, void* k_cache, void* v_cache, const int32_t* cu_q,
                         const int32_t* ctx_lens, const int32_t* tok_seq, const int32_t* block_tables,
                         int bt_stride, int64_t T, int H, int G, int D, int Dv, int page, float eps, int dtype,
                         void* stream);

/* Pooled entry of block b (positions bP .. bP+P-1) lives with the page of its last token:
 * kp [pages, ceil(page/P), G, D], vp [pages, ceil(page/P), G, Dv], local index b - floor(page*j/P) in page j.
 * Computes the blocks completed by this step; max_new_blocks bounds them per sequence. */
int lv_pool_update(const void* k_cache, const void* v_cache, void* kp, void* vp, const int32_t* cu_q,
                   const int32_t* ctx_lens, const int32_t* block_tables, int bt_stride, int B, int max_new_blocks,
                   int G, int D, int Dv, int page, int P, int dtype, void* stream);

/* Query at position i sees cached positions j with 0 <= i-j < window and every pooled block b with
 * b*P + P - 1 <= i - window (P == 0: no pooled blocks); weights exp(s) / (sink + sum exp(s)) with
 * sink = 1 for has_sink, else 0.  gate (optional) act rows of stride ld_gate holding H*Dv numbers
 * (LV_MIX_GATE_PER_CHANNEL) or H (LV_MIX_GATE_PER_HEAD): out *= sigmoid(gate).
 * q act [T, H*D] contiguous; out act [T, H*Dv].  k_ld, v_ld: elements between two tokens' rows in k_cache and v_cache
 * (0: G*D and G*Dv); the pooled caches are always dense. */
int lv_window_pool_attn(const void* q, const void* k_cache, const void* v_cache, const void* kp, const void* vp,
                        const void* gate, int64_t ld_gate, void* out, const int32_t* cu_q, const int32_t* ctx_lens,
                        const int32_t* tok_seq, const int32_t* block_tables, int bt_stride, int64_t T, int H, int G,
                        int D, int Dv, int page, int window, int P, float scale, int has_sink, int64_t k_ld,
                        int64_t v_ld, int gate_kind, int dtype, void* stream);

/* The same attention on the matrix cores: bf16 only, D and Dv multiples of 16 up to 256. Tiles of 16 new
 * tokens per sequence; max_new_tokens = the largest cu_q[b+1] - cu_q[b] of the step.
 * nsplit > 1 (only with max_new_tokens <= 16, i.e. decode-shaped steps): the key tiles of a sequence are cut over nsplit
 * workgroups whose partials a second kernel merges; workspace: f32 [T, H, nsplit, Dv + 4] (read-out, maximum, sum, padding), T = total new tokens. */
int lv_window_pool_attn_mfma(const void* q, const void* k_cache, const void* v_cache, const void* kp, const void* vp,
                             const void* gate, int64_t ld_gate, void* out, const int32_t* cu_q, const int32_t* ctx_lens,
                             const int32_t* block_tables, int bt_stride, int B, int max_new_tokens, int H, int G, int D,
                             int Dv, int page, int window, int P, float scale, int has_sink, int nsplit, void* workspace,
                             int64_t T, int64_t k_ld, int64_t v_ld, int gate_kind, void* stream);

/* Latent attention, step 1. proj act [T, ld]: the query latent at column off_q (Rq wide), the key/value latent at
 * off_kv (R wide) directly followed by the positional key part (Dr wide, may be 0).
 * cq_out act [T, Rq] = rms_norm(query latent) * q_w.  cache act [pages, page, R + Dr]: the row of each token's position
 * receives rms_norm(latent) * kv_w | rotated positional part.  Rotation: of the first rot_dims (even, <= Dr) entries,
 * entry i pairs with i + rot_dims/2, angle = position * inv_freq[i] (inv_freq f32 [rot_dims/2]). */
int lv_latent_prep(const void* proj, int64_t ld, int off_q, int off_kv, const void* q_w, const void* kv_w,
                   const void* inv_freq, void* cq_out, void* cache, const int32_t* cu_q, const int32_t* ctx_lens,
                   const int32_t* tok_seq, const int32_t* block_tables, int bt_stride, int64_t T, int Rq, int R, int Dr,
                   int rot_dims, int page, float eps, int dtype, void* stream);

/* Latent attention, step 2. q act [T, H, Dn + Dr] (the rotated part last), q_lat act [H, T, R] (the unrotated part
 * already multiplied into the latent space).  q_out act [T, H, R + Dr] = q_lat | rotate(q[.., Dn:], position). */
int lv_latent_q_finish(const void* q, const void* q_lat, const void* inv_freq, void* q_out, const int32_t* cu_q,
                       const int32_t* ctx_lens, const int32_t* tok_seq, int64_t T, int H, int Dn, int Dr, int R,
                       int rot_dims, int dtype, void* stream);

/* o act [H, T, Dv] -> out act [T, H*Dv] = o * sigmoid(gate); gate act rows of stride ld_gate holding H numbers
 * (LV_MIX_GATE_PER_HEAD) or H*Dv (LV_MIX_GATE_PER_CHANNEL). */
int lv_latent_out_gate(const void* o, const void* gate, int64_t ld_gate, int gate_kind, void* out, int64_t T, int H,
                       int Dv, int dtype, void* stream);

/* Router of a mixture of experts. logits f32 [T, E]; scores s = sigmoid(logits); selection scores c = s + correction
 * (f32 [E], may be NULL). The experts are split into `groups` consecutive blocks of equal size; a block is ranked by its
 * two highest selection scores added up (by its one, for blocks of one expert); experts outside the `keep` highest-ranked blocks are excluded
 * (groups <= 1: all). The `top` largest c are chosen (ties: lowest index first); weights = their s / (sum + 1e-20),
 * or their s as they are when `normalize` is 0.
 * ids int32 [T, top], weights f32 [T, top], dense f32 [T, E] (weights at the chosen experts, 0 elsewhere; may be NULL). */
int lv_moe_route(const void* logits, const void* correction, void* ids, void* weights, void* dense, int64_t T, int E,
                 int top, int groups, int keep, int normalize, void* stream);

/* Router logits of steps of few tokens: logits f32 [T, E] = router_w h in f32 (h act [T, W] with row stride ld_h, router_w
 * f32 [E, W]), without a widened copy of h; one workgroup per (token, four experts). */
int lv_router_logits(const void* h, int64_t ld_h, const void* router_w, void* logits, int64_t T, int W, int E, int dtype,
                     void* stream);

/* up act [T, E*F] (all experts' up projections side by side), dense f32 [T, E]:
 * out act [T, E*F] = relu(up)^2 * dense[t, e]. */
int lv_relu2_scale(const void* up, const void* dense, void* out, int64_t T, int E, int F, int dtype, void* stream);

/* The gathered form of the same feed-forward, bf16 only, W and F multiples of 32: the (token, choice) pairs are sorted by
 * expert on the device, each expert multiplies its own rows on the matrix cores (up projection with relu^2, down
 * projection), and every token sums its choices' rows times their weights in f32. Four launches, no host round trip.
 * h bf16 [T, W]; ids int32 [T, top]; weights f32 [T, top]; up_w bf16 [E*F, W]; down_w bf16 [W, E*F]; out bf16 [T, W];
 * workspace: lv_moe_grouped_workspace_bytes(T, W, F, E, top) bytes, 16-byte aligned. */
int lv_moe_grouped_ff(const void* h, const void* ids, const void* weights, const void* up_w, const void* down_w, void* out,
                      void* workspace, int64_t T, int W, int F, int E, int top, void* stream);
int64_t lv_moe_grouped_workspace_bytes(int64_t T, int W, int F, int E, int top);

/* The sort and the weighted sum of the gathered form on their own, for callers that multiply the sorted rows themselves.
 * ids int32 [M] (expert of pair p = token * top + choice) -> sorted_pair int32 (pair of each row in expert order),
 * inv int32 [M] (row of each pair), offsets int32 [E + 1] (first row of each expert). Every expert's rows start on a
 * multiple of `align`, so an expert owns rows [offsets[e], offsets[e + 1]), the last ones of which may be padding that the
 * kernel does not write: sorted_pair has room for M + E * align entries and is cleared by the caller. */
int lv_moe_sort(const void* ids, int64_t M, int E, int align, void* sorted_pair, void* inv, void* offsets, void* stream);
/* rows bf16 [M, W] (expert outputs in sorted order), inv int32 [T, top], weights f32 [T, top] (NULL: all one):
 * out bf16 [T, W] = sum_k weights[t, k] * rows[inv[t, k]] in f32; W a multiple of 4. */
int lv_moe_combine(const void* rows, const void* inv, const void* weights, void* out, int64_t T, int W, int top, void* stream);


/* x f32 [T, W] in place:  x += y / sqrt(mean(y^2) + eps) * (w_offset + post_w)   (y act [T, W] with post_w f32 [W]; both NULL: skipped)
 *                         x += rows + vec                                         (rows act [T, W], vec f32 [W]; either may be NULL)
 * out act [T, W] = x / sqrt(mean(x^2) + eps) * (w_offset + w)  (out and w may be NULL: update only). All arithmetic f32. */
int lv_sandwich_add_norm(void* x, const void* y, const void* post_w, const void* rows, const void* vec, const void* w,
                         float w_offset, void* out, int64_t T, int W, float eps, int dtype, void* stream);

/* proj act [T, ld]: H query heads of D at column off_q, G key heads of D at off_k, G value heads of Dv at off_v.
 * The first rot_dims (even, <= D) entries of every query and key head are rotated: entry i pairs with i + rot_dims/2,
 * angle = position * inv_freq[i] (f32 [rot_dims/2]), position = ctx_lens[b] + index in the step; query head h is then
 * multiplied by head_scale[h] (f32 [H], may be NULL).  q_out act [T, H*D] contiguous; rotated keys into
 * k_cache [pages, page, G, D] and values into v_cache [pages, page, G, Dv] at the token's slot. */
int lv_rotary_store(const void* proj, int64_t ld, int off_q, int off_k, int off_v, const void* inv_freq,
                    const void* head_scale, void* q_out, void* k_cache, void* v_cache, const int32_t* cu_q,
                    const int32_t* ctx_lens, const int32_t* tok_seq, const int32_t* block_tables, int bt_stride, int64_t T,
                    int H, int G, int D, int Dv, int rot_dims, int page, int dtype, void* stream);

/* in act [T, F] (row stride ld_in), coef f32 [4] = c1, c2, c3, c0:
 * out act [T, F] = c1 z / rms(z) + c2 z^2 / rms(z^2) + c3 z^3 / rms(z^3) + c0, rms(u) = sqrt(mean_F(u^2) + eps), f32. */
int lv_polynorm(const void* in, int64_t ld_in, const void* coef, void* out, int64_t T, int F, float eps, int dtype,
                void* stream);

/* in act [T, E*2F] (row stride ld_in), expert e's columns = [gate F | up F]; in_scale f32 [T, E] or NULL (all one);
 * out_gate act, a scalar for each token at stride ld_gate, or NULL.
 * s = in_scale[t, e]; g = min(s * gate, limit); u = clamp(s * up, -limit, limit);
 * out act [T, E*F] (row stride ld_out) = g * sigmoid(alpha * g) * (u + 1) * sigmoid(out_gate[t]); 0 where s == 0. */
int lv_expert_glu(const void* in, int64_t ld_in, const void* in_scale, const void* out_gate, int64_t ld_gate, void* out,
                  int64_t ld_out, int64_t T, int E, int F, float limit, float alpha, int dtype, void* stream);

/* lv_moe_grouped_ff for clamped gated experts: up_w bf16 [E*2F, W] (per expert F gate rows, then F up rows),
 * down_w bf16 [W, E*F] with row stride down_ld (0: E*F; a column block of a wider weight otherwise).
 * out[t] = sum_k W_down,e glu(weights[t, k] * W_gu,e h[t]), e = ids[t, k]: the weight scales the expert's input and the
 * outputs are summed as they are. Workspace: lv_moe_grouped_workspace_bytes(T, W, F, E, top) bytes, 16-byte aligned. */
int lv_moe_grouped_glu_ff(const void* h, const void* ids, const void* weights, const void* up_w, const void* down_w,
                          int64_t down_ld, void* out, void* workspace, int64_t T, int W, int F, int E, int top, float limit,
                          float alpha, void* stream);

/* x f32 [T, W] in place.  post_w1 == NULL:  x += y1 + y2                  (act [T, W]; either may be NULL)
 *                         post_w1 != NULL:  x += pair_scale * (y1 / rms(y1) * post_w1 + y2 / rms(y2) * post_w2)
 *                                           (rms(y) = sqrt(mean(y^2) + eps); y2 with post_w2 may be NULL)
 * out act [T, W] = tanh(alpha[0] * x) * w + b  (alpha f32 [1], w and b f32 [W]; out may be NULL: update only). All f32. */
int lv_residual_dyt(void* x, const void* y1, const void* post_w1, const void* y2, const void* post_w2, float pair_scale,
                    float eps, const void* alpha, const void* w, const void* b, void* out, int64_t T, int W, int dtype,
                    void* stream);

/* lv_rotary_store with two more choices. interleaved != 0: rotated entry 2i pairs with 2i + 1 (else i with i + rot_dims/2),
 * angle = position * inv_freq[i]. unit_norm != 0: every query and key head is divided by sqrt(mean(head^2) + eps) (no weight). */
int lv_qk_prep_store(const void* proj, int64_t ld, int off_q, int off_k, int off_v, const void* inv_freq,
                     const void* head_scale, void* q_out, void* k_cache, void* v_cache, const int32_t* cu_q,
                     const int32_t* ctx_lens, const int32_t* tok_seq, const int32_t* block_tables, int bt_stride, int64_t T,
                     int H, int G, int D, int Dv, int rot_dims, int interleaved, int unit_norm, float eps, int page, int dtype,
                     void* stream);

/* lv_window_pool_attn with more ways to say what a query at position i sees among the cached positions j <= i:
 *   chunk == 0: i - j < window or j < keep_first;   chunk > 0: floor(i / chunk) == floor(j / chunk) or j < keep_first
 * (kept first tokens and chunks do not combine with pooled blocks, P > 0). sinks f32 [H] (may be NULL): the denominator of
 * head h's softmax also holds exp(sinks[h]); has_sink without sinks: exp(0). */
int lv_masked_attn(const void* q, const void* k_cache, const void* v_cache, const void* kp, const void* vp,
                   const void* gate, int64_t ld_gate, void* out, const int32_t* cu_q, const int32_t* ctx_lens,
                   const int32_t* tok_seq, const int32_t* block_tables, int bt_stride, int64_t T, int H, int G, int D,
                   int Dv, int page, int window, int keep_first, int chunk, int P, float scale, int has_sink,
                   const void* sinks, int64_t k_ld, int64_t v_ld, int gate_kind, int dtype, void* stream);
int lv_masked_attn_mfma(const void* q, const void* k_cache, const void* v_cache, const void* kp, const void* vp,
                        const void* gate, int64_t ld_gate, void* out, const int32_t* cu_q, const int32_t* ctx_lens,
                        const int32_t* block_tables, int bt_stride, int B, int max_new_tokens, int H, int G, int D,
                        int Dv, int page, int window, int keep_first, int chunk, int P, float scale, int has_sink,
                        const void* sinks, int nsplit, void* workspace, int64_t T, int64_t k_ld, int64_t v_ld,
                        int gate_kind, void* stream);

/* proj act [T, ld]: H query heads of D at column off_q, H key heads of D at off_k, H value heads of Dv at off_v; each entry
 * passes silu first. Per head and token: S <- decay[h] * S + k v^T; o = S^T q. state f32 [slots, H, D, Dv], read unless
 * ctx_lens[b] == 0, written back; decay f32 [H]; o f32 [T, H, Dv]. */
int lv_lightning_attn(const void* proj, int64_t ld, int off_q, int off_k, int off_v, const void* decay, void* state,
                      const int32_t* cu_q, const int32_t* ctx_lens, const int32_t* slots, void* o, int B, int H, int D, int Dv,
                      int dtype, void* stream);

/* in act [T, 2F] (row stride ld_in) = [gate | up];  out act [T, F] = act(gate) * up, act one of LV_MIX_ACT_*. */
int lv_glu_act(const void* in, int64_t ld_in, void* out, int64_t T, int F, int act, int dtype, void* stream);

/* lv_moe_route with the scores as sigmoid or as softmax over all E logits of the row (LV_MIX_SCORE_*), and the rank of a
 * group as the sum of its two highest selection scores or its highest (LV_MIX_GROUP_*). */
int lv_moe_route_scored(const void* logits, const void* correction, void* ids, void* weights, void* dense, int64_t T, int E,
                        int top, int groups, int keep, int normalize, int score_kind, int group_rank, void* stream);

/* up act [T, E*F], dense f32 rows of stride ld_dense (>= E):  out act [T, E*F] = act(up) * dense[t, e], 0 where dense is 0. */
int lv_expert_act_scale(const void* up, const void* dense, int64_t ld_dense, void* out, int64_t T, int E, int F, int act,
                        int dtype, void* stream);

/* lv_moe_grouped_ff with the activation as a choice and n_through more expert numbers (E_real .. E_real + n_through - 1)
 * that stand for no weights: such a choice contributes weight * h[t]. ids hold numbers below E_real + n_through;
 * workspace: lv_moe_grouped_workspace_bytes(T, W, F, E_real + n_through, top). */
int lv_moe_grouped_act_ff(const void* h, const void* ids, const void* weights, const void* up_w, const void* down_w, void* out,
                          void* workspace, int64_t T, int W, int F, int E_real, int n_through, int top, int act, void* stream);
/* lv_moe_combine in which a choice with ids[t, k] >= n_real takes the row h[t] (bf16 [T, W]) instead of a row of `rows`. */
int lv_moe_combine_through(const void* rows, const void* inv, const void* weights, void* out, int64_t T, int W, int top,
                           const void* ids, int n_real, const void* h, void* stream);

/* y act [T, W] += (factors[t, 0] + ... + factors[t, nf - 1]) * h[t]; factors f32 rows of stride ld_f. */
int lv_scaled_row_add(void* y, const void* h, const void* factors, int64_t ld_f, int nf, int64_t T, int W, int dtype,
                      void* stream);

#ifdef __cplusplus
}
#endif
#endif
