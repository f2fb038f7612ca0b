/* C ABI of the layer-list ("hybrid") host layer: decoder-only models whose config lists, layer by layer, which token mixer a
 * layer has -- sliding-window attention with a softmax sink, a gated delta rule (recurrent matrix state), a minGRU (recurrent vector
 * state), attention and delta rule side by side, latent attention (keys and values read off one cached latent vector per token), or
 * attention behind a short convolution whose heads' softmax weights are mixed -- and which feed-forward (dense gate/up forms or a
 * mixture of experts), or a state-space mixer with a scalar decay per head.  The Sogodra, Vivazen, Kerolorn and Sabolorn designs are
 * its users.
 *
 * What differs from the llama-family host layers (mi355_llama_*, mi355_dense_*):
 *   - the residual stream, norms, attention scores, decays, gates of a recurrence and the recurrent state are f32 in both dtypes;
 *     `dtype` = MI355_DTYPE_BF16 keeps the matrices (and the K/V pages) in bf16 and multiplies on the matrix cores with f32
 *     accumulation, MI355_DTYPE_F32 keeps everything in f32 and multiplies with plain f32 FMAs (no reduced-precision mode);
 *   - one step function for prompts, portions of prompts and single decoded tokens: every sequence of a step brings
 *     cu_seqlens_q[i+1] - cu_seqlens_q[i] new tokens behind context_lens[i] - that many cached ones (the fields of
 *     mi355_be_prepare_prompt); K/V live in the block engine's pages, recurrent state in the block engine's state slots
 *     (mi355_be_state_*), one slot per live sequence;
 *   - a sequence whose portion starts at position 0 starts from zero state whatever its slot held before.
 * Every entry point returns 0 on success (hipError_t or a negative argument error otherwise) and only enqueues work on `stream`. */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_HYB_MIX_PARALLEL 0   /* attention ("left") and gated delta rule ("right") on the same input, outputs scaled and added */
#define MI355_HYB_MIX_MINGRU 1
#define MI355_HYB_MIX_DELTA 2
#define MI355_HYB_MIX_ATTENTION 3  /* the attention branch alone */
#define MI355_HYB_MIX_LATENT 4     /* latent attention: the pages hold [latent c (a_kv_rank) | rotated key part (a_rot_dim)] per token;
                                      head h's key is W_uk,h c and its value W_uv,h c.  Computed in the absorbed form: the query
                                      carries W_uk,h^T q_h, the attention runs over the latent rows themselves (one shared key/value
                                      head of a_kv_rank + a_rot_dim / a_kv_rank dimensions), W_uv,h is applied to its output */
#define MI355_HYB_MIX_CONV_ATTENTION 5 /* q, k, v pass a short causal convolution (a_conv taps, no activation), then attention with
                                      the a_* switches below; the convolution's last inputs live in the state slot */

#define MI355_HYB_MIX_SSD 6         /* selective state-space mixer (scalar decay per head): the input projection gives [gate z | x | B | C |
                                      step dt]; x, B, C pass a short causal convolution with bias and silu; per head S <- exp(-exp(a_log)
                                      dt) S + dt B x^T, y = S^T C + skip x; y silu(z), RMS norm in d_norm_groups parts, output projection.
                                      d_heads heads of d_vdim, state size d_dim, d_kv_heads groups of B / C, d_conv taps            */

#define MI355_HYB_GATE_SILU 0      /* output gate silu(W_g h), full rank                */
#define MI355_HYB_GATE_SIGMOID_LR 1 /* output gate sigmoid(W_g2 (W_g1 h)), low rank     */

typedef struct mi355_hybrid_layer {
    int32_t mixer;                 /* MI355_HYB_MIX_*                                                              */
    /* attention branch */
    int32_t a_heads, a_kv_heads, a_dim, a_vdim;
    int32_t a_window;              /* 0 = none; else a query at position i sees keys j with 0 <= i - j < a_window  */
    int32_t a_rot_dims;            /* leading dimensions of a head that are rotated (rotate-half pairs), 0 = none  */
    int32_t a_has_sink;            /* the softmax denominator also holds exp(sink[head])                           */
    int32_t a_qk_norm;             /* RMS norm of every query / key head before the rotation                       */
    float a_scale, a_out_scale;
    /* delta-rule branch */
    int32_t d_heads, d_kv_heads, d_dim, d_vdim, d_conv;
    int32_t d_decay_channels;      /* 0: one decay per head (full-rank W_a [heads, width]);
                                      1: one per head and key channel (low rank W_a2 (W_a1 h), rank d_a_rank)      */
    int32_t d_a_rank;
    int32_t d_gate;                /* MI355_HYB_GATE_*                                                             */
    int32_t d_g_rank;
    float d_out_scale;
    /* minGRU */
    int32_t g_width;
    /* feed-forward: 0 = none, 1 = dense clamped gate/up with y = g sigmoid(act_alpha g) (u + 1),
                     2 = dense gate/up with y = gelu_tanh(g) u,
                     3 = mixture of experts with y = silu(g) u (fields below; the shared expert, when there is one, uses the dense
                         slots MI355_HW_MLP_GATE_UP / _DOWN with moe_shared_ff)                                       */
    int32_t mlp_kind, mlp_ff;
    float mlp_limit, mlp_alpha;
    /* more switches of the attention branch (all 0 = the plain form) */
    int32_t a_rot_interleaved;     /* rotated pairs are (2i, 2i + 1) instead of (i, i + a_rot_dims / 2)                   */
    int32_t a_kv_rank, a_rot_dim;  /* latent attention: latent size; rotated dimensions per query head = the shared key part
                                      (a_dim = the unrotated dimensions per head, a_rot_dims <= a_rot_dim of them turn)    */
    int32_t a_head_gate;           /* head h's output times sigmoid((W_g x)_h), W_g [heads, width] in the input projection */
    int32_t a_conv;                /* taps of the convolution behind q, k, v                                               */
    int32_t a_norm_whole;          /* a_qk_norm is ONE RMS norm over all of q (and of k), weights [heads * dim]            */
    int32_t a_v_unit;              /* every value head is divided by its root mean square before it is cached             */
    float a_softcap;               /* > 0: score <- cap tanh(score / cap)                                                  */
    int32_t a_talk;                /* weight_h <- sum_g talk[h, g] weight_g after the softmax; head h applies its mixed
                                      weights to the values of its own key/value head                                      */
    int32_t share_with;            /* 0: the layer has weights; n > 0: it runs on layer n - 1's weights (and rope tables) with
                                      pages and state of its own                                                           */
    /* switches of the plain attention mixers (MI355_HYB_MIX_ATTENTION / _PARALLEL), all 0 = the form above */
    int32_t a_keep_first;          /* with a window: keys at positions < a_keep_first stay visible to every later query     */
    int32_t a_norm_after_rot;      /* the RMS norm of q and k (a_qk_norm) is taken AFTER the rotation and has no weight     */
    int32_t a_head_temp;           /* head h's scores are multiplied by temp[h] (MI355_HW_A_TEMP)                           */
    /* input convolution in front of the mixer: what the mixer reads, h, becomes h + conv(h), a causal convolution over time on
     * every channel of the width (in_conv taps, 0 = none); the last taps - 1 rows of h live in the state slot                  */
    int32_t in_conv;
    /* feed-forward kind 3, a mixture of experts: moe_experts gate/up experts of mlp_ff with silu, every token uses the moe_top with
     * the largest softmax(router) + correction; its weights are the chosen experts' softmax values times moe_scale (not
     * renormalised).  moe_shared_ff > 0: one more expert of that size runs for every token, times sigmoid(w_sg . h)              */
    int32_t moe_experts, moe_top, moe_shared_ff;
    float moe_scale;
    /* more switches of the router (all 0 = the form above) */
    int32_t moe_sigmoid;           /* scores are sigmoid(z) instead of softmax(z)                                           */
    int32_t moe_groups, moe_keep_groups; /* > 0: the experts form moe_groups equal groups of neighbours; a group's score is the sum of
                                      its two largest choice scores and only experts of the best moe_keep_groups groups can be chosen */
    int32_t moe_normalise;         /* the chosen experts' scores are divided by their sum (+ 1e-20) before moe_scale         */
    /* feed-forward kind 4: dense without a gate, y = W_down relu(W_up h)^2 (MI355_HW_MLP_GATE_UP holds the [ff, width] up rows)  */
    int32_t d_norm_groups;         /* MI355_HYB_MIX_SSD: parts of the gated output with a root mean square of their own      */
    int32_t a_dist_bias;           /* MI355_HYB_MIX_CONV_ATTENTION: score <- score - r1[h] ln(1 + r2[h] (i - j)), MI355_HW_A_DIST */
    int32_t a_q_rank;              /* latent attention, > 0: queries through a latent, q = W_uq RMSnorm(W_dq h) (MI355_HW_L_UQ,
                                      MI355_HW_L_QNORM); the q part of the input projection then holds the a_q_rank rows of W_dq */
    int32_t a_out_gate;            /* latent attention: the concatenated heads times sigmoid(W_g h) element by element, W_g
                                      [heads vdim, width] in the gate part of the input projection                            */
    int32_t kv_from;               /* latent attention, n > 0: no down-projection and no pages of its own; the layer reads the pages
                                      that layer n - 1 (an earlier latent layer of the same kv_rank / rot_dim) has written       */
    int32_t side_dim;              /* > 0: after the sublayers x <- x + RMSnorm(W_proj (gelu_tanh(W_gate x) * e)) w with e = the
                                      token's row of the side table, columns [side_col, side_col + side_dim)                   */
    int32_t side_col;
    int32_t depth_terms;           /* n > 0: behind the layer x <- sum_j w[j] X_j over the n earliest of (embedding output, results
                                      of the layers so far); n = layer index + 2 (MI355_HW_DEPTH_W [n])                        */
} mi355_hybrid_layer;

typedef struct mi355_hybrid_config {
    int32_t width, vocab, n_layers;
    int32_t dtype;                 /* MI355_DTYPE_F32 or MI355_DTYPE_BF16                                          */
    int32_t block_size;            /* tokens per K/V page                                                          */
    int32_t state_slots;           /* recurrent-state slots (live sequences)                                       */
    float norm_eps;
    float unit_eps;                /* eps inside the root of the unit norm of q and k in the delta rule            */
    int32_t residual_form;         /* 0: x <- x + norm(sub(x));  1: x <- norm(resid_alpha x + sub(x));
                                      2: x <- x + norm(sub(pre_norm(x))), a norm on both sides of every sublayer
                                         (MI355_HW_PRE_NORM1 / 2 in front, MI355_HW_NORM1 / 2 behind)                 */
    float resid_alpha;
    int32_t norm_groups;           /* the layer norms and the last norm take the RMS over this many equal consecutive parts
                                      of the vector separately (0 or 1: over the whole vector)                       */
    float logit_scale;             /* the logits are multiplied by it (0 = 1)                                        */
    /* residual_form 3: ONE norm per layer, h = norm(x) (MI355_HW_NORM1), and both sublayers read it: x <- x + mixer(h) + ff(h) */
    int32_t norm_kind;             /* 0: RMS norm; 1: layer norm with a weight and no bias, (x - mean) / sqrt(var + eps) w -- the
                                      norm in front of the sublayers (form 3) and the last norm                              */
    float embed_scale;             /* the embedding rows are multiplied by it (0 = 1)                                        */
    float logit_softcap;           /* > 0: logits <- cap tanh(logits / cap)                                                  */
    int32_t tie_head;              /* the logits are taken against the embedding table itself; MI355_HW_HEAD stays empty     */
    int32_t side_cols;             /* columns of the per-layer token table MI355_HW_SIDE_TABLE [vocab, side_cols] (0 = none) */
} mi355_hybrid_config;

/* weight slots: `layer` = -1 for the three global ones */
#define MI355_HW_EMBED 0           /* [vocab, width]                                                                */
#define MI355_HW_FINAL_NORM 1      /* [width]                                                                       */
#define MI355_HW_HEAD 2            /* [vocab, width]                                                                */
#define MI355_HW_NORM1 3           /* [width]  norm on the mixer's output                                           */
#define MI355_HW_NORM2 4           /* [width]  norm on the feed-forward's output                                    */
#define MI355_HW_IN_PROJ 5         /* every projection that reads the mixer's input, concatenated along the rows in
                                      the order of mi355_hybrid_in_proj_rows: [rows, width]                         */
#define MI355_HW_IN_BIAS 6         /* [rows] or absent                                                              */
#define MI355_HW_OUT_PROJ 7        /* [width, k]: the output projections side by side along k (attention first)     */
#define MI355_HW_A_QNORM 8
#define MI355_HW_A_KNORM 9
#define MI355_HW_A_SINK 10
#define MI355_HW_D_CONV 11         /* [q channels + k channels + v channels, taps], last column = the current token */
#define MI355_HW_D_A_LOG 12        /* [heads]                                                                       */
#define MI355_HW_D_DT_BIAS 13      /* [heads] or [heads * dim]                                                      */
#define MI355_HW_D_NORM 14         /* [vdim]                                                                        */
#define MI355_HW_D_A2 15           /* [heads * dim, a_rank]                                                         */
#define MI355_HW_D_G2 16           /* [heads * vdim, g_rank]                                                        */
#define MI355_HW_MLP_GATE_UP 17    /* [2 ff, width]: gate rows, then up rows                                        */
#define MI355_HW_MLP_DOWN 18       /* [width, ff]                                                                   */
#define MI355_HW_A_CONV 19         /* [q channels + k channels + v channels, taps], last column = the current token */
#define MI355_HW_A_TALK 20         /* [heads, heads]                                                                */
#define MI355_HW_L_UKT 21          /* [heads, kv_rank, dim]: per head the TRANSPOSE of its block of W_uk [heads dim, kv_rank] */
#define MI355_HW_L_UV 22           /* [heads vdim, kv_rank]                                                         */
#define MI355_HW_L_CNORM 23        /* [kv_rank] weight of the latent's RMS norm                                      */
#define MI355_HW_PRE_NORM1 24      /* [width]  residual form 2: norm in front of the mixer                           */
#define MI355_HW_PRE_NORM2 25      /* [width]  residual form 2: norm in front of the feed-forward                    */
#define MI355_HW_IN_CONV 26        /* [width, in_conv], last column = the current token                              */
#define MI355_HW_A_TEMP 27         /* [heads]                                                                        */
#define MI355_HW_MOE_ROUTER 28     /* f32 [experts (+ 1 when moe_shared_ff: the shared expert's gate row last), width] */
#define MI355_HW_MOE_CORRECTION 29 /* [experts] added to the softmax values for the choice only                      */
#define MI355_HW_MOE_GATE_UP 30    /* [experts, 2 ff, width]: per expert gate rows, then up rows; a shared expert of the
                                      experts' size (moe_shared_ff == mlp_ff) is one more matrix at the end, here and in
                                      MOE_DOWN, and the dense slots stay empty                                       */
#define MI355_HW_MOE_DOWN 31       /* [experts, width, ff]                                                           */
#define MI355_HW_D_SKIP 32         /* [heads]  state-space mixer: y += skip[h] x                                     */
#define MI355_HW_CONV_BIAS 33      /* [channels] bias of the convolution MI355_HW_D_CONV                             */
#define MI355_HW_A_DIST 34         /* [2, heads]: r1, then r2 of the distance bias                                   */
#define MI355_HW_L_QNORM 35        /* [q_rank] weight of the query latent's RMS norm                                 */
#define MI355_HW_L_UQ 36           /* [heads (dim + rot_dim), q_rank]                                                */
#define MI355_HW_SIDE_GATE 37      /* [side_dim, width]                                                              */
#define MI355_HW_SIDE_PROJ 38      /* [width, side_dim]                                                              */
#define MI355_HW_SIDE_NORM 39      /* [width]                                                                        */
#define MI355_HW_DEPTH_W 40        /* [depth_terms]                                                                  */
#define MI355_HW_COUNT 41
#define MI355_HW_SIDE_TABLE 41     /* global (layer -1): [vocab, side_cols]                                          */

void* mi355_hybrid_create(const mi355_hybrid_config* cfg, const mi355_hybrid_layer* layers);
void mi355_hybrid_destroy(void* model);
/* rows of a layer's concatenated input projection, and where each part starts: parts = attention q, k, v, delta q, k, v, beta,
 * decay (a or a1), gate (g or g1) for the attention / delta / parallel mixers; z, x, g for the minGRU; q (heads x (dim + rot_dim)),
 * the latent down-projection (kv_rank + rot_dim) in the k part and the head gate in the gate part for latent attention.
 * offsets[9], -1 = absent */
int32_t mi355_hybrid_in_proj_rows(const mi355_hybrid_layer* layer, int32_t* offsets);
/* HOST bf16 bits (a checkpoint tensor), n elements; converted to the storage type of the slot */
int mi355_hybrid_set_weight(void* model, int32_t layer, int32_t which, const uint16_t* host_bf16, int64_t n);
/* DEVICE bf16 bits (synthetic weights of a benchmark) */
int mi355_hybrid_set_weight_dev(void* model, int32_t layer, int32_t which, const uint16_t* dev_bf16, int64_t n, int64_t stream);
/* HOST f32 [n_positions, a_rot_dims / 2] cos and sin of a layer's rotary angles (mi355_rope_tables builds them) */
int mi355_hybrid_set_rope_tables(void* model, int32_t layer, const float* cos_t, const float* sin_t, int32_t n_positions);
/* K/V pages of every attention layer and the state pool; all state starts as zero */
int mi355_hybrid_alloc_cache(void* model, int32_t num_blocks);
int64_t mi355_hybrid_cache_bytes(void* model, int32_t num_blocks);
int64_t mi355_hybrid_state_floats_per_slot(void* model);
void* mi355_hybrid_state_ptr(void* model);
/* one step over DEVICE inputs.  tokens u32 [T]; positions, slot_mapping i64 [T]; block_tables u32 [num_seqs, max_blocks];
 * context_lens u32 [num_seqs] (cached + new); cu_seqlens_q u32 [num_seqs + 1]; state_slots i32 [num_seqs]; out_rows i32 [n_out]
 * = the token rows whose logits are wanted -> logits f32 [n_out, vocab].  layer_trace: NULL, or f32 [n_layers, T, width] that
 * receives the residual stream behind every layer (parity hook). */
int mi355_hybrid_forward(void* model, const uint32_t* tokens, const int64_t* positions, const int64_t* slot_mapping,
                         const uint32_t* block_tables, const uint32_t* context_lens, const uint32_t* cu_seqlens_q,
                         const int32_t* state_slots, const int32_t* out_rows, int32_t n_out, int32_t num_seqs, int32_t num_tokens,
                         int32_t max_blocks, int32_t max_context_len, float* logits, float* layer_trace, int64_t stream);

/* the same step from a hipGraph keyed by the device pointers and the counts (the caller keeps its step inputs in static device
 * buffers); `stream` must not be the default stream; no layer trace */
int mi355_hybrid_forward_graph(void* model, const uint32_t* tokens, const int64_t* positions, const int64_t* slot_mapping,
                               const uint32_t* block_tables, const uint32_t* context_lens, const uint32_t* cu_seqlens_q,
                               const int32_t* state_slots, const int32_t* out_rows, int32_t n_out, int32_t num_seqs,
                               int32_t num_tokens, int32_t max_blocks, int32_t max_context_len, float* logits, int64_t stream);
int64_t mi355_hybrid_graph_captures(void* model);
int64_t mi355_hybrid_graph_replays(void* model);

/* ---- the mechanisms alone (tests, other host layers).  `dtype` is the type of 16/32-bit operands marked (dt); the rest is f32 */
/* token_seq i32 [T]: the sequence (row of cu_seqlens_q) of every token row */
int mi355_hyb_token_seq(int32_t* token_seq, const uint32_t* cu_seqlens_q, int32_t num_seqs, int64_t stream);
int mi355_hyb_bf16_to_f32(float* out, const uint16_t* in, int64_t n, int64_t stream);
int mi355_hyb_copy_f32(float* out, const float* in, int64_t n, int64_t stream);
int mi355_hyb_fill_f32(float* out, float v, int64_t n, int64_t stream);
/* x f32 [T, width] = table (dt) [vocab, width] rows ids; xcopy: NULL or bf16 [T, width] */
int mi355_hyb_embed(float* x, void* xcopy, const void* table, const uint32_t* ids, int32_t num_tokens, int32_t width, int32_t vocab,
                    int32_t dtype, int64_t stream);
/* out (dt_out) [n_rows, width] = RMS norm with weight of the rows `rows` of x */
int mi355_hyb_gather_norm(void* out, int32_t out_dtype, const float* x, const int32_t* rows, const float* w, int32_t n_rows,
                          int32_t width, float eps, int64_t stream);
/* out f32 [T, ldo] = a (dt_a: F32 or BF16) [T, lda] . w (dt) [n, k]^T + bias f32 [n] */
int mi355_hyb_linear(float* out, int32_t ldo, const void* a, int32_t a_dtype, int32_t lda, const void* w, const float* bias,
                     int32_t num_tokens, int32_t n, int32_t k, int32_t dtype, int64_t stream);
/* x f32 [T, width] += y / rms(y) * w, y f32 [T, ldy]; xcopy (NULL or bf16 [T, width]) receives the rounded sum */
int mi355_hyb_norm_add(float* x, void* xcopy, const float* y, int32_t ldy, const float* w, int32_t num_tokens, int32_t width,
                       float eps, int64_t stream);
/* per-head RMS norm (weights NULL = none) and rotation of q / k out of the projection rows, q -> q_out (dt) [T, heads, dim],
 * k, v -> the pages at slot_mapping (dt), [blocks, block_size, kv_heads, dim | vdim] */
int mi355_hyb_attn_prepare(void* q_out, void* k_pages, void* v_pages, const float* proj, int32_t ldp, int32_t q_off, int32_t k_off,
                           int32_t v_off, const float* q_norm_w, const float* k_norm_w, const float* cos_t, const float* sin_t,
                           const int64_t* positions, const int64_t* slot_mapping, int32_t num_tokens, int32_t heads,
                           int32_t kv_heads, int32_t dim, int32_t vdim, int32_t rot_dims, float eps, int32_t dtype, int64_t stream);
/* causal attention of every new token over its sequence's pages: window (0 = none), sink f32 [heads] or NULL;
 * out (dt_out) [T, ldo] at column out_off: heads x vdim, times out_scale */
int mi355_hyb_window_attention(void* out, int32_t out_dtype, int32_t ldo, int32_t out_off, const void* q, const void* k_pages,
                               const void* v_pages, const uint32_t* block_tables, const uint32_t* context_lens,
                               const uint32_t* cu_seqlens_q, const int32_t* token_seq, const float* sink, int32_t num_seqs, int32_t num_tokens,
                               int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, int32_t block_size, int32_t max_blocks,
                               int32_t window, float scale, float out_scale, int32_t dtype, int64_t stream);
/* the same with the remaining switches: k_ld / v_ld = elements per page row of the key / value pages (0: kv_heads x dim | vdim;
 * latent attention passes the same pages for both with v_ld = k_ld), softcap (0 = none), cross_values: 1 = every query head's
 * weights are applied to the values of EVERY key/value head c, out [T, heads, kv_heads, vdim] (what mi355_hyb_head_mix reads) */
int mi355_hyb_window_attention_ex(void* out, int32_t out_dtype, int32_t ldo, int32_t out_off, const void* q, const void* k_pages,
                                  const void* v_pages, const uint32_t* block_tables, const uint32_t* context_lens,
                                  const uint32_t* cu_seqlens_q, const int32_t* token_seq, const float* sink, int32_t num_seqs,
                                  int32_t num_tokens, int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, int32_t block_size,
                                  int32_t max_blocks, int32_t window, float scale, float out_scale, int32_t k_ld, int32_t v_ld,
                                  float softcap, int32_t cross_values, int32_t dtype, int64_t stream);
/* out (dt_out) [T, heads x vdim] = sum_g talk[h, g] a[t, g, kv head of h, :],  a f32 [T, heads, kv_heads, vdim]: mixing the heads'
 * softmax weights before the value product is the same as mixing, per key/value head, the outputs the unmixed weights give */
int mi355_hyb_head_mix(void* out, int32_t out_dtype, const float* a, const float* talk, int32_t num_tokens, int32_t heads,
                       int32_t kv_heads, int32_t vdim, int64_t stream);
/* out (dt_out) [T, heads x vdim] = in f32 [T, heads x vdim] times sigmoid(gate_in[t, h]) per head (gate_in NULL: a plain copy) */
int mi355_hyb_head_gate(void* out, int32_t out_dtype, const float* in, const float* gate_in, int32_t ldg, int32_t num_tokens,
                        int32_t heads, int32_t vdim, int64_t stream);
/* attention behind a convolution: src f32 [T, ld] holds q | k | v rows (offsets q_off, k_off, v_off).  q and k: RMS norm over the WHOLE
 * row part (heads x dim, kv_heads x dim) with weights of that size (NULL = no norm); v: every head divided by its root mean square when
 * v_unit.  q -> q_out (dt) [T, heads, dim], k, v -> the pages at slot_mapping.  No rotation */
int mi355_hyb_attn_prepare_whole(void* q_out, void* k_pages, void* v_pages, const float* src, int32_t ld, int32_t q_off, int32_t k_off,
                                 int32_t v_off, const float* q_norm_w, const float* k_norm_w, const int64_t* slot_mapping,
                                 int32_t num_tokens, int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, int32_t v_unit, float eps,
                                 int32_t dtype, int64_t stream);
/* latent attention: proj f32 [T, ldp] holds per head [dim unrotated | rot_dim rotated] query rows at q_off and the down-projection
 * [kv_rank | rot_dim] at c_off; q_abs f32 [T, heads, kv_rank] = the unrotated query parts already multiplied by W_uk^T.
 * pages (dt) [.., kv_rank + rot_dim] at slot_mapping <- [RMS norm of the latent times c_norm_w | rotated key part];
 * q_out (dt) [T, heads, kv_rank + rot_dim] <- [q_abs | rotated query part].  The first rot_dims of the rot_dim dimensions turn
 * (pairs (2i, 2i+1) when interleaved), cos_t / sin_t [positions, rot_dims / 2] carry any amplitude */
int mi355_hyb_latent_prepare(void* q_out, void* pages, const float* proj, int32_t ldp, int32_t q_off, int32_t c_off, const float* q_abs,
                             const float* c_norm_w, const float* cos_t, const float* sin_t, const int64_t* positions,
                             const int64_t* slot_mapping, int32_t num_tokens, int32_t heads, int32_t dim, int32_t rot_dim,
                             int32_t kv_rank, int32_t rot_dims, int32_t interleaved, float eps, int32_t dtype, int64_t stream);
/* `batch` independent products of one shape in one launch: out + z o_bs [T, ldo] = (a + z a_bs) [T, lda] . (w + z w_bs) [n, k]^T,
 * strides in elements (per-head matrices: z = head) */
int mi355_hyb_linear_batched(float* out, int32_t ldo, int64_t o_bs, const void* a, int32_t a_dtype, int32_t lda, int64_t a_bs,
                             const void* w, int64_t w_bs, int32_t num_tokens, int32_t n, int32_t k, int32_t batch, int32_t dtype,
                             int64_t stream);
/* x f32 [T, width] <- group norm(alpha x + y) times w (the norm BEHIND the residual sum; `groups` equal consecutive parts, each with
 * its own root mean square); xcopy: NULL or bf16 [T, width] */
int mi355_hyb_resid_norm(float* x, void* xcopy, const float* y, int32_t ldy, const float* w, int32_t num_tokens, int32_t width,
                         int32_t groups, float alpha, float eps, int64_t stream);
/* mi355_hyb_gather_norm with the RMS taken over `groups` parts */
int mi355_hyb_gather_group_norm(void* out, int32_t out_dtype, const float* x, const int32_t* rows, const float* w, int32_t n_rows,
                                int32_t width, int32_t groups, float eps, int64_t stream);
/* out (dt_out) [T, ff] = gelu_tanh(gu[:, j]) gu[:, ff + j] */
int mi355_hyb_gelu_glu(void* out, int32_t out_dtype, const float* gu, int32_t num_tokens, int32_t ff, int64_t stream);
/* mi355_hyb_conv_silu with the activation as an argument: 0 = none, 1 = silu */
int mi355_hyb_conv(float* out, const float* proj, int32_t ldp, int32_t off, const float* w, const float* conv_state,
                   int64_t state_stride, const uint32_t* context_lens, const uint32_t* cu_seqlens_q, const int32_t* state_slots,
                   const int32_t* token_seq, int32_t num_seqs, int32_t num_tokens, int32_t channels, int32_t taps, int32_t act,
                   int64_t stream);
/* ---- mechanisms of the pre/post-norm designs */
/* out (dt_out) [T, width] = RMS norm of every row of x times w (the norm in front of a sublayer) */
int mi355_hyb_pre_norm(void* out, int32_t out_dtype, const float* x, const float* w, int32_t num_tokens, int32_t width, float eps,
                       int64_t stream);
/* out (dt_out) [T, channels] = h + conv(h) for h = in f32 [T, ld] columns [off, off + channels): the causal convolution of
 * mi355_hyb_conv added to its own input; mi355_hyb_conv_state_update(in) then moves the state behind the portion */
int mi355_hyb_conv_residual(void* out, int32_t out_dtype, const float* in, int32_t ld, int32_t off, const float* w,
                            const float* conv_state, int64_t state_stride, const uint32_t* context_lens, const uint32_t* cu_seqlens_q,
                            const int32_t* state_slots, const int32_t* token_seq, int32_t num_seqs, int32_t num_tokens, int32_t channels,
                            int32_t taps, int64_t stream);
/* the two above in ONE launch for taps <= 8: h = RMS norm of x times norm_w (norm_w NULL: h = x), out (dt_out) [T, width] = h + conv(h).
 * hn: NULL, or f32 [T, width] that receives h (what mi355_hyb_conv_state_update then reads).  update_state != 0 (only when every
 * sequence brings one token, T == num_seqs): the kernel moves the state behind the token itself and no update launch is needed */
int mi355_hyb_norm_conv(void* out, int32_t out_dtype, float* hn, const float* x, const float* norm_w, const float* conv_w, float* conv_state,
                        int64_t state_stride, const uint32_t* context_lens, const uint32_t* cu_seqlens_q, const int32_t* state_slots,
                        const int32_t* token_seq, int32_t num_seqs, int32_t num_tokens, int32_t width, int32_t taps, int32_t update_state,
                        float eps, int64_t stream);
/* mi355_hyb_attn_prepare with the remaining switches: interleaved = rotated pairs are (2i, 2i + 1); norm_mode 0 = none, 1 = RMS norm
 * with weights before the rotation (q_norm_w / k_norm_w, NULL = no weight), 2 = RMS norm without a weight AFTER the rotation;
 * q_head_scale f32 [heads] or NULL: head h's query is multiplied by it (a temperature per head folded into the query) */
int mi355_hyb_attn_prepare_ex(void* q_out, void* k_pages, void* v_pages, const float* proj, int32_t ldp, int32_t q_off, int32_t k_off,
                              int32_t v_off, const float* q_norm_w, const float* k_norm_w, const float* cos_t, const float* sin_t,
                              const int64_t* positions, const int64_t* slot_mapping, int32_t num_tokens, int32_t heads,
                              int32_t kv_heads, int32_t dim, int32_t vdim, int32_t rot_dims, int32_t interleaved, int32_t norm_mode,
                              const float* q_head_scale, float eps, int32_t dtype, int64_t stream);
/* mi355_hyb_window_attention_ex with kept first tokens: beside the keys inside its window (all earlier keys when window == 0) a query
 * sees the keys at positions below keep_first; those keep their own positions and rotations */
int mi355_hyb_masked_attention(void* out, int32_t out_dtype, int32_t ldo, int32_t out_off, const void* q, const void* k_pages,
                               const void* v_pages, const uint32_t* block_tables, const uint32_t* context_lens,
                               const uint32_t* cu_seqlens_q, const int32_t* token_seq, const float* sink, int32_t num_seqs,
                               int32_t num_tokens, int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, int32_t block_size,
                               int32_t max_blocks, int32_t window, int32_t keep_first, float scale, float out_scale, int32_t k_ld,
                               int32_t v_ld, float softcap, int32_t cross_values, int32_t dtype, int64_t stream);
/* mixture of experts, routing: h = RMS norm of x times norm_w (norm_w NULL: h = x) -> xn (dt_out) [T, width] (NULL = not written);
 * z = router f32 [experts, width] . h in f32, s = softmax(z); the `top` experts with the largest s + correction (correction NULL =
 * none; ties to the lower expert) -> expert_ids i32 [T, top] in descending order of the choice score, weights f32 [T, top] =
 * s[chosen] * scale.  gate_row f32 [width] or NULL: shared_gate f32 [T] (NULL = not written) = sigmoid(gate_row . h).
 * append_shared: expert_ids and weights are [T, top + 1] and every token's last pair is (expert `experts`, that sigmoid): a shared
 * expert of the experts' size runs as one more group of the grouped products */
int mi355_hyb_moe_route(int32_t* expert_ids, float* weights, float* shared_gate, void* xn, int32_t out_dtype, const float* x,
                        const float* norm_w, const float* router, const float* correction, const float* gate_row, int32_t num_tokens,
                        int32_t width, int32_t experts, int32_t top, float scale, float eps, int32_t append_shared, int64_t stream);
/* rows of a grouped product's blocks that suit `pairs` (token, expert) pairs over `experts` experts with [n, k] matrices: 16 (few
 * rows per expert: a stream over the weights), 64 or 128 (matrix-core tiles through LDS) */
int32_t mi355_hyb_moe_block_rows(int32_t pairs, int32_t experts, int32_t n, int32_t k, int32_t dtype);
/* grouping on the device: every expert owns whole blocks of block_rows rows of the gathered buffers, expert e's rows start at
 * block_rows * (blocks of the experts before it).  pos i32 [pairs] = the row of pair p = token * top + slot; row_token i32 [n_blocks *
 * block_rows] = the token of every used row; block_table i32 [n_blocks, 2] = {expert, one past the expert's last row} for every block
 * ({0, 0} past the last expert's), n_blocks >= ceil(pairs / block_rows) + experts */
int mi355_hyb_moe_group(int32_t* pos, int32_t* row_token, int32_t* block_table, const int32_t* expert_ids, int32_t pairs, int32_t top,
                        int32_t experts, int32_t block_rows, int32_t n_blocks, int64_t stream);
/* one product per block of the table: out f32 rows [b block_rows, block end) = a rows . (w + expert w_bs) [n, k]^T; a (dt_a) [.., lda]
 * row r is read at row_token[r] when row_token != NULL (gathered from the token rows), else at r */
int mi355_hyb_linear_grouped(float* out, int32_t ldo, const void* a, int32_t a_dtype, int32_t lda, const int32_t* row_token,
                             const void* w, int64_t w_bs, const int32_t* block_table, int32_t block_rows, int32_t n_blocks, int32_t n,
                             int32_t k, int32_t dtype, int64_t stream);
/* out (dt_out) [rows, ff] = silu(gu[:, j]) gu[:, ff + j]; block_table != NULL: only the rows that a block of the table uses */
int mi355_hyb_silu_glu(void* out, int32_t out_dtype, const float* gu, int32_t rows, int32_t ff, const int32_t* block_table,
                       int32_t block_rows, int64_t stream);
/* x f32 [T, width] += y / rms(y) * w with y[t] = sum_j weights[t, j] y_rows[pos[t top + j]] + shared_gate[t] y_shared[t]
 * (y_shared NULL = no shared expert; shared_gate NULL = 1); xcopy: NULL or bf16 [T, width] */
int mi355_hyb_moe_combine_norm_add(float* x, void* xcopy, const float* y_rows, const int32_t* pos, const float* weights,
                                   const float* y_shared, const float* shared_gate, const float* w, int32_t num_tokens, int32_t width,
                                   int32_t top, float eps, int64_t stream);
int mi355_hyb_scale_f32(float* x, float s, int64_t n, int64_t stream);
/* ---- mechanisms of the parallel-residual designs (hybrid_blocks.hip) */
/* x f32 [T, width] = table rows ids times scale */
int mi355_hyb_embed_scaled(float* x, const void* table, const uint32_t* ids, int32_t num_tokens, int32_t width, int32_t vocab, float scale,
                           int32_t dtype, int64_t stream);
/* out (dt_out) [T, width] (and out_f32, NULL or f32 [T, width]) = norm of the rows of x f32 [T, ldx] times w; kind 0: RMS, 1: layer
 * norm (mean taken off, variance = mean of the squared deviations) */
int mi355_hyb_pre_norm_ex(void* out, int32_t out_dtype, float* out_f32, const float* x, int32_t ldx, const float* w, int32_t num_tokens,
                          int32_t width, int32_t kind, float eps, int64_t stream);
/* mi355_hyb_gather_norm with the kind of norm as an argument */
int mi355_hyb_gather_norm_ex(void* out, int32_t out_dtype, const float* x, const int32_t* rows, const float* w, int32_t n_rows,
                             int32_t width, int32_t kind, float eps, int64_t stream);
/* x f32 [T, width] += a + b (b NULL: += a) */
int mi355_hyb_add2(float* x, const float* a, const float* b, int64_t n, int64_t stream);
/* x[t] += y[t] + sum_j weights[t, j] y_rows[pos[t top + j]]  (y NULL = none): the experts' weighted sum without a norm */
int mi355_hyb_moe_combine_add(float* x, const float* y, const float* y_rows, const int32_t* pos, const float* weights, int32_t num_tokens,
                              int32_t width, int32_t top, int64_t stream);
/* out (dt_out) [T, ff] = relu(u)^2 */
int mi355_hyb_relu2(void* out, int32_t out_dtype, const float* u, int64_t n, int64_t stream);
/* x <- cap tanh(x / cap) */
int mi355_hyb_tanh_cap(float* x, float cap, int64_t n, int64_t stream);
/* out (dt_out) [T, n] = in f32 [T, n] times sigmoid(gate_in[t, c]) element by element, gate_in f32 rows of ldg */
int mi355_hyb_elem_gate(void* out, int32_t out_dtype, const float* in, const float* gate_in, int32_t ldg, int32_t num_tokens, int32_t n,
                        int64_t stream);
/* out (dt_out) [T, dim] = gelu_tanh(g[t, k]) * table (dt) [vocab, ldt] row ids[t], column col + k */
int mi355_hyb_side_act(void* out, int32_t out_dtype, const float* g, const void* table, int32_t ldt, int32_t col, const uint32_t* ids,
                       int32_t num_tokens, int32_t dim, int32_t vocab, int32_t dtype, int64_t stream);
/* xs f32 [terms, n]: xs[terms - 1] <- x (the newest result), then x <- sum_j w[j] xs[j] */
int mi355_hyb_depth_average(float* x, float* xs, const float* w, int32_t terms, int64_t n, int64_t stream);
/* the end of a layer and the start of the next in one launch: x += y / rms(y) * side_w (y NULL: nothing added); then, with depth_w,
 * mi355_hyb_depth_average over xs; then, with norm_w, out (dt_out) [T, width] (and out_f32, NULL or f32) = the norm of kind `kind` of
 * the new x times norm_w (what mi355_hyb_pre_norm_ex would give) */
int mi355_hyb_layer_tail(float* x, const float* y, const float* side_w, float* xs, const float* depth_w, int32_t terms, void* out, int32_t out_dtype,
                         float* out_f32, const float* norm_w, int32_t num_tokens, int32_t width, int32_t kind, float eps, int64_t stream);
/* out (dt_out) [T, n] = (y * silu(gate_in[t, c])) / rms over each of `groups` equal parts * w[c]: the gate in front of the norm */
int mi355_hyb_gate_group_norm(void* out, int32_t out_dtype, const float* y, const float* gate_in, int32_t ldg, const float* w,
                              int32_t num_tokens, int32_t n, int32_t groups, float eps, int64_t stream);
/* state-space scan over the new tokens of every sequence, state f32 [slots] x [heads, n_state, vdim] (stride in floats).
 * xbc f32 [T, ldx]: x (heads x vdim) at 0, B (groups x n_state) behind it, C behind that, all behind the convolution and silu;
 * dt_in f32 rows of ldd: the raw step per head; dt = softplus(dt_in + dt_bias[h]), decay = exp(-exp(a_log[h]) dt);
 * S <- decay S + dt B x^T;  y f32 [T, heads, vdim] = S^T C + skip[h] x.  Head h reads group h / (heads / groups).  n_state <= 512. */
int mi355_hyb_ssd_scan(float* y, float* state, int64_t state_stride, const float* xbc, int32_t ldx, const float* dt_in, int32_t ldd,
                       const float* a_log, const float* dt_bias, const float* skip, const uint32_t* context_lens,
                       const uint32_t* cu_seqlens_q, const int32_t* state_slots, int32_t num_seqs, int32_t num_tokens, int32_t heads,
                       int32_t groups, int32_t n_state, int32_t vdim, int64_t stream);
/* mi355_hyb_conv with a bias per channel (NULL = none) in front of the activation */
int mi355_hyb_conv_bias(float* out, const float* proj, int32_t ldp, int32_t off, const float* w, const float* bias, const float* conv_state,
                        int64_t state_stride, const uint32_t* context_lens, const uint32_t* cu_seqlens_q, const int32_t* state_slots,
                        const int32_t* token_seq, int32_t num_seqs, int32_t num_tokens, int32_t channels, int32_t taps, int32_t act,
                        int64_t stream);
/* mi355_hyb_masked_attention with a distance bias: dist f32 [2, heads] (NULL = none), score <- score - r1[h] ln(1 + r2[h] (i - j)) */
int mi355_hyb_biased_attention(void* out, int32_t out_dtype, int32_t ldo, int32_t out_off, const void* q, const void* k_pages,
                               const void* v_pages, const uint32_t* block_tables, const uint32_t* context_lens,
                               const uint32_t* cu_seqlens_q, const int32_t* token_seq, const float* sink, const float* dist,
                               int32_t num_seqs, int32_t num_tokens, int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim,
                               int32_t block_size, int32_t max_blocks, int32_t window, int32_t keep_first, float scale, float out_scale,
                               int32_t k_ld, int32_t v_ld, float softcap, int32_t cross_values, int32_t dtype, int64_t stream);
/* mi355_hyb_latent_prepare with the query rows and the down-projection in buffers of their own: q_src f32 [T, ldq] holds per head
 * [dim | rot_dim] at q_off; c_src f32 [T, ldc] holds [kv_rank | rot_dim] at c_off.  pages NULL: nothing is cached (a layer that reads
 * another layer's pages) and c_src is not read */
int mi355_hyb_latent_prepare_ex(void* q_out, void* pages, const float* q_src, int32_t ldq, int32_t q_off, const float* c_src, int32_t ldc,
                                int32_t c_off, const float* q_abs, const float* c_norm_w, const float* cos_t, const float* sin_t,
                                const int64_t* positions, const int64_t* slot_mapping, int32_t num_tokens, int32_t heads, int32_t dim,
                                int32_t rot_dim, int32_t kv_rank, int32_t rot_dims, int32_t interleaved, float eps, int32_t dtype,
                                int64_t stream);
/* mi355_hyb_moe_route with the remaining switches: sigmoid_scores (s = sigmoid(z) instead of softmax), groups / keep_groups (> 0: only
 * experts of the keep_groups groups with the largest sum of their two best choice scores can be chosen), normalise (weights divided
 * by their sum + 1e-20 before the scale) */
int mi355_hyb_moe_route_ex(int32_t* expert_ids, float* weights, float* shared_gate, void* xn, int32_t out_dtype, const float* x,
                           const float* norm_w, const float* router, const float* correction, const float* gate_row, int32_t num_tokens,
                           int32_t width, int32_t experts, int32_t top, float scale, float eps, int32_t append_shared,
                           int32_t sigmoid_scores, int32_t groups, int32_t keep_groups, int32_t normalise, int64_t stream);
/* 0: prompt-sized steps over bf16 pages take the generic kernel instead of the matrix-core ones; 2: the matrix-core kernel with one
 * wave per head also where the query heads of a key/value head could share a workgroup (A/B switch, process-wide; default 1) */
void mi355_hyb_set_attention_mfma(int32_t on);
/* short causal convolution over time per channel, then silu: out f32 [T, channels] from proj columns [off, off + channels);
 * the taps - 1 inputs before a portion come from conv_state f32 [slots, channels, taps - 1] (zeros at position 0);
 * mi355_hyb_conv_state_update then moves the state behind the portion */
int mi355_hyb_conv_silu(float* out, const float* proj, int32_t ldp, int32_t off, const float* w, const float* conv_state,
                        int64_t state_stride, const uint32_t* context_lens, const uint32_t* cu_seqlens_q,
                        const int32_t* state_slots, const int32_t* token_seq, int32_t num_seqs, int32_t num_tokens, int32_t channels,
                        int32_t taps, int64_t stream);
int mi355_hyb_conv_state_update(float* conv_state, int64_t state_stride, const float* proj, int32_t ldp, int32_t off,
                                const uint32_t* context_lens, const uint32_t* cu_seqlens_q, const int32_t* state_slots,
                                int32_t num_seqs, int32_t channels, int32_t taps, int64_t stream);
/* gated delta rule over the new tokens of every sequence, state f32 [slots] x [heads, dim, vdim] (stride in floats).
 * qkv f32 [T, ldq]: q at 0 (kv_heads x dim, raw), k behind it, v behind that (heads x vdim); q and k are made unit vectors per head
 * (eps inside the root), q times dim^-1/2.  beta = sigmoid(proj[:, b_off + head]).  decay = exp(-exp(a_log[head]) * softplus(da +
 * dt_bias)) with da = decay_in[t, head] (channels = 0) or decay_in[t, head * dim + channel].  o f32 [T, heads, vdim]. */
int mi355_hyb_delta_rule(float* o, float* state, int64_t state_stride, const float* qkv, int32_t ldq, const float* proj,
                         int32_t ldp, int32_t b_off, const float* decay_in, int32_t ldd, int32_t decay_channels,
                         const float* a_log, const float* dt_bias, const uint32_t* context_lens, const uint32_t* cu_seqlens_q,
                         const int32_t* state_slots, int32_t num_seqs, int32_t num_tokens, int32_t heads, int32_t kv_heads, int32_t dim,
                         int32_t vdim, float unit_eps, float* scratch, int64_t stream);
/* floats of `scratch` (device): what the rule computes for all tokens at once before the scan over them */
int mi355_hyb_delta_rule_scratch_floats(int32_t num_tokens, int32_t heads, int32_t kv_heads, int32_t dim, int32_t decay_channels);
/* out (dt_out) [T, ldo] at out_off = o / rms(o over vdim) * w * gate(gate_in) * out_scale; gate: MI355_HYB_GATE_* (silu / sigmoid) */
int mi355_hyb_gated_norm(void* out, int32_t out_dtype, int32_t ldo, int32_t out_off, const float* o, const float* w,
                         const float* gate_in, int32_t ldg, int32_t gate, int32_t num_tokens, int32_t heads, int32_t vdim, float eps,
                         float out_scale, int64_t stream);
/* minGRU over the new tokens: z = sigmoid(proj[:, z_off + c]), u = proj[:, x_off + c], candidate = u + 1/2 (u >= 0) or sigmoid(u),
 * S = (1 - z) S + z candidate, out (dt_out) [T, width] = S silu(proj[:, g_off + c]); state f32 [slots] x [width] */
int mi355_hyb_mingru(void* out, int32_t out_dtype, float* state, int64_t state_stride, const float* proj, int32_t ldp, int32_t z_off,
                     int32_t x_off, int32_t g_off, const uint32_t* context_lens, const uint32_t* cu_seqlens_q,
                     const int32_t* state_slots, int32_t num_seqs, int32_t num_tokens, int32_t width, int64_t stream);
/* out (dt_out) [T, ff] = g sigmoid(alpha g) (u + 1), g = min(gu[:, j], limit), u = clamp(gu[:, ff + j], -limit, limit) */
int mi355_hyb_clamped_glu(void* out, int32_t out_dtype, const float* gu, int32_t num_tokens, int32_t ff, float limit, float alpha,
                          int64_t stream);

#ifdef __cplusplus
}
#endif
