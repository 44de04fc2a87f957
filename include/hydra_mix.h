/*
 * hydra_mix.h — C ABI of libhydra_mix.so: kernels of the sequence-mixing mechanisms that the Llama path does not have —
 * multi-stream residuals (hyper-connections) with grouped RMS norm, token shift and gated sublayer results, the tanh
 * GELU gate, and attention over a paged cache of low-rank latents (one latent row per token, shared by all heads) with a
 * sliding window; and, for depth-averaged recurrent / attention hybrids: token + learned position embedding, layer
 * norms around every sublayer with the residual kept in a stack of levels (depth-weighted average), the PolyNorm and
 * squared-ReLU activations, a softmax router with a choice bias, grouped expert products over expert-major rows, a
 * gated linear recurrence with a matrix state per head (HGRN2), and grouped-query attention over a paged key/value
 * cache with a per-head linear distance bias, an optional soft cap on the scores and a causal, windowed or chunked mask;
 * and, for mixers that keep per-sequence state beside the cache: short causal convolutions, token shift with several
 * mixes, per-head RMS norm + rotary positions + cache append, decays / step sizes / write strengths of a recurrence, a scan
 * over a matrix state per head in three forms (decayed sum, read-before-write with a bonus, delta rule), the gate / group
 * norm that finishes a mixer, and a clamped gated feed-forward activation; and, for attention with sinks: a learned extra
 * term in the softmax's denominator and a temperature per head (both attention kernels), rotary positions over parts of a
 * token's row in either pair layout with values that turn too (hxm_rotary_parts), two short convolutions of one input
 * added to it, identity experts and un-renormalised router weights.
 *
 * Same conventions as hydra_hip.h: raw device pointers, sizes and strides in ELEMENTS, a hipStream_t passed as void*,
 * asynchronous launches, no allocation, 0 or a negative hx_status (hydra_hip.h) as the result.  `dtype` is the hx_dtype
 * of the ACTIVATIONS (what the matrix products read and write): HX_F32 or HX_BF16.  The residual streams, the per-sequence
 * state, norm / shift / mixing weights and biases are always float.
 *
 * The library is separate from libhydra_hip.so so that a model that needs only these kernels builds only these.
 */
#ifndef HYDRA_MIX_H
#define HYDRA_MIX_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HXM_ABI_VERSION 4
#define HXM_MAX_STREAMS 16
#define HXM_MAX_LATENT 1024     /* widest latent row the attention kernels hold in registers (the MFMA tile form: 512) */

int hxm_abi_version(void);
int hxm_last_hip_error(void);
/* A/B measurements in one process: "attn_tile_form" = 0 keeps bfloat16 attention on the row form (one wave per token
 * and head) instead of the MFMA forms, 2 keeps portions of prompts on the tile form (one wave per 16 rows) instead of
 * the group form (four waves sharing every chunk of keys), 1 = the default.  Results agree within bfloat16 rounding. */
int hxm_set_option(const char* name, int value);

/* x[t, s, :] = table[ids[t], :] * scale for every stream s.  x: float [n_tokens, n_streams, width]; table: dtype
 * [vocab, width]; ids: int32 or int64.  An id outside [0, vocab) writes zeros. */
int hxm_stream_embed(float* x, const void* table, const void* ids, int ids_are_int64, float scale, int64_t n_tokens,
                     int32_t n_streams, int64_t width, int64_t vocab, int dtype, void* stream);

/* The input of a sublayer: u = sum_s in_w[s] * x[row, s, :], h = u / sqrt(mean_group(u^2) + eps) * norm_w over `groups`
 * equal consecutive groups.  rows (optional): int32 [n_out] rows of x to take (output row i <- x row rows[i]); else
 * output row i <- x row i.  h_out: dtype [n_out, width] (may be NULL when only the shifted form is wanted).
 *
 * Token shift (shift_w != NULL; rows must be NULL): hs = h + (h_prev - h) * shift_w, h_prev = the h of the token before
 * in the same sequence: the previous row of the batch, or — for the first token of a sequence's portion — the row that
 * the sequence's state slot holds (zeros at position 0).  The slot then receives the h of the portion's last token.
 * state: float, slot s at state + s * state_slot_stride (width floats).  tok_seq: int32 [n_tokens] sequence of each
 * token; q_cu: int32 [n_seq + 1]; positions: int32 [n_tokens]; slots: int32 [n_seq]. */
int hxm_stream_norm(const float* x, const float* in_w, const float* norm_w, int32_t groups, float eps,
                    const int32_t* rows, int64_t n_out, int32_t n_streams, int64_t width, void* h_out,
                    const float* shift_w, void* hs_out, float* state, int64_t state_slot_stride,
                    const int32_t* tok_seq, const int32_t* q_cu, const int32_t* positions, const int32_t* slots,
                    int dtype, void* stream);

/* A sublayer's result enters the streams: g = y * sigmoid(gate_pre + gate_b) (gate_pre == NULL: g = y), then for every
 * target stream t: x[., t, :] <- sum_s mix[s * n_streams + t] * x[., s, :] + out_w[t] * g, all targets from the old
 * values.  y: dtype [n_tokens, >= width] with row stride y_stride; gate_pre likewise; gate_b: float [width] or NULL. */
int hxm_stream_update(float* x, const void* y, int64_t y_stride, const void* gate_pre, int64_t gate_stride,
                      const float* gate_b, const float* mix, const float* out_w, int64_t n_tokens, int32_t n_streams,
                      int64_t width, int dtype, void* stream);

/* hxm_stream_update followed by the read side of the NEXT sublayer (one without a token shift) in one launch: the streams
 * are updated in place and h_out [n_tokens, width] = grouped_rms_norm(sum_s in_next[s] * x_new[., s, :]) * norm_next. */
int hxm_stream_update_norm(float* x, const void* y, int64_t y_stride, const void* gate_pre, int64_t gate_stride,
                           const float* gate_b, const float* mix, const float* out_w, const float* in_next,
                           const float* norm_next, int32_t groups, float eps, void* h_out, int64_t n_tokens,
                           int32_t n_streams, int64_t width, int dtype, void* stream);

/* out[., i] = gelu_tanh(gate[., i]) * up[., i], gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))). */
int hxm_gelu_tanh_and_mul(void* out, const void* gate, const void* up, int64_t rows, int64_t n, int64_t gate_stride,
                          int64_t up_stride, int dtype, void* stream);

/* The two latents of a token from one projection row: cq = rms_norm(proj[., q_off : q_off + q_rank]) * q_w -> cq_out
 * [n_tokens, q_rank]; c = rms_norm(proj[., kv_off : kv_off + kv_rank]) * kv_w -> the paged cache at slot_ids[token]
 * (slot = block * block_size + row; slots < 0 are skipped).  cache: dtype, block b at cache + b * cache_block_stride, row r
 * of it cache_row_stride further.  Plain (one group) RMS norms with eps inside the root. */
int hxm_latent_norm_cache(const void* proj, int64_t proj_stride, int64_t q_off, int64_t q_rank, int64_t kv_off,
                          int64_t kv_rank, const float* q_w, const float* kv_w, float eps, void* cq_out,
                          const int32_t* slot_ids, void* cache, int64_t cache_block_stride, int64_t cache_row_stride,
                          int32_t block_size, int64_t n_tokens, int dtype, void* stream);

typedef struct hxm_latent_attn_args {
  void* out;                 /* dtype [n_tokens, n_heads, kv_rank] (strides below): sum_j p_j c_j, times the head gate */
  const void* q;             /* dtype [n_tokens, n_heads, kv_rank]: the queries already carried into the latent space */
  const void* cache;         /* dtype paged latents */
  const void* gate_pre;      /* dtype, optional: out is multiplied by sigmoid(gate_pre[t * gate_stride + head]) */
  const int32_t* tok_seq;    /* [n_tokens] */
  const int32_t* positions;  /* [n_tokens] position of each query in its sequence (= its own key's index) */
  const int32_t* q_cu;       /* [n_seq + 1] */
  const int32_t* block_table;/* flat */
  const int32_t* cu_block_lens; /* [n_seq + 1] */
  int64_t q_token_stride, q_head_stride, out_token_stride, out_head_stride, gate_stride;
  int64_t cache_block_stride, cache_row_stride;
  int32_t n_tokens, n_seq, n_heads, kv_rank, block_size;
  int32_t window;            /* a query at position i sees keys j with 0 <= i - j < window; <= 0: every j <= i */
  int32_t max_q_len;         /* the longest portion of the batch (1: every sequence decodes) */
  float scale;
  int32_t dtype;
  int32_t max_kv_len;        /* the most keys a sequence of the batch holds (sizes the key splits) */
  int32_t n_splits;          /* from hxm_latent_attention_plan; > 1: the key range of a row tile is dealt to n_splits waves */
  float* ws_o;               /* n_splits > 1: the plan's workspace, ws_floats floats; ws_ml = where its (max, sum) pairs go */
  float* ws_ml;
  const float* sinks;        /* [n_heads] or NULL: the softmax's denominator of head h holds one more term exp(sinks[h]), which
                                has no key and no value (an attention sink); it is not scaled */
} hxm_latent_attn_args;

/* How a launch with these arguments would be laid out: n_splits (1: no workspace) and the floats of workspace it needs
 * (ws_o = the first n_items * n_splits * 16 * ceil16(kv_rank) of them, ws_ml = the rest).  Pointers need not be set yet,
 * except q and cache (their alignment decides the form). */
int hxm_latent_attention_plan(const hxm_latent_attn_args* args, int32_t* n_splits, int64_t* ws_floats);

/* Softmax attention of every query over the latents of its own sequence in the paged cache (scores and weights in
 * float).  Queries of portions and single decoded tokens may share a batch. */
int hxm_latent_attention(const hxm_latent_attn_args* args, void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Depth-averaged residual with layer norms (hxm_depth_norm), embeddings, activations.
 * ------------------------------------------------------------------------------------------------------------------ */

/* out[t, :] = table[ids[t], :] + pos_table[positions[t], :] in float (pos_table may be NULL).  table, pos_table: dtype.
 * An id outside [0, vocab) or a position outside [0, n_positions) contributes zeros. */
int hxm_embed_positions(float* out, const void* table, const void* pos_table, const void* ids, int ids_are_int64,
                        const int32_t* positions, int64_t n_tokens, int64_t width, int64_t vocab, int64_t n_positions,
                        int dtype, void* stream);

/* One row kernel for every place where a residual meets a norm.  LN(u) = (u - mean(u)) / sqrt(var(u) + eps), var the mean
 * squared deviation; with rms != 0: LN(u) = u / sqrt(mean(u^2) + eps).  For output row i (input row r = rows ? rows[i] : i):
 *   x = x_in ? x_in[r] : 0
 *   if y:         x += mult * N(y[r]) * post_w                       (a sublayer's result enters the residual; N by post_norm:
 *                                                                     LN as above, the layer norm, the RMS norm, or y as it is —
 *                                                                     then post_w may be NULL: ones)
 *   if y2:        x += y2[r]                                         (a second sublayer that read the same input)
 *   if bias:      x += bias                                          (a float vector of `width`)
 *   if level_out: level_out[r] = x                                   (the layer's own result joins the stack of levels)
 *   if depth_w:   x = sum_{j < n_levels} depth_w[j] * levels[j][r]   (levels[j] = levels + j * level_stride; may include
 *                                                                     the level just written)
 *   if x_out:     x_out[i] = x
 *   if next_w:    h_out[i] = LN(x) * next_w                          (dtype; the next sublayer's input)
 *   else if h_out: h_out[i] = x                                      (dtype; the residual as a matrix product's operand)
 * x_in, level_out, levels, x_out: float rows of `width` (contiguous).  y, y2: dtype, row strides y_stride, y2_stride; h_out:
 * dtype, row stride h_stride (so that it may be a column range of a wider matrix). */
#define HXM_POST_SAME 0     /* y is normed like everything else in the call (rms) */
#define HXM_POST_LAYER 1    /* layer norm */
#define HXM_POST_RMS 2      /* RMS norm */
#define HXM_POST_PLAIN 3    /* no norm */
typedef struct hxm_depth_norm_args {
  const float* x_in;
  const void* y;
  const float* post_w;
  float* level_out;
  const float* levels;
  const float* depth_w;
  float* x_out;
  const float* next_w;
  void* h_out;
  const int32_t* rows;
  int64_t y_stride, level_stride, n_out, width;
  int32_t n_levels, rms, dtype;
  float mult, eps;
  const void* y2;
  const float* bias;
  int64_t y2_stride, h_stride;
  int32_t post_norm;         /* HXM_POST_* */
} hxm_depth_norm_args;
int hxm_depth_norm(const hxm_depth_norm_args* args, void* stream);

/* PolyNorm: out = c[0] N(z) + c[1] N(z^2) + c[2] N(z^3) + c[3], powers element by element, N(u) = u / sqrt(mean(u^2) + eps)
 * over the row.  coef: float[4] on the device.  z, out: dtype [rows, n] with their row strides. */
int hxm_poly_norm(void* out, int64_t out_stride, const void* z, int64_t z_stride, const float* coef, float eps, int64_t rows,
                  int64_t n, int dtype, void* stream);

/* out = max(z, 0)^2 */
int hxm_relu_squared(void* out, int64_t out_stride, const void* z, int64_t z_stride, int64_t rows, int64_t n, int dtype,
                     void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Mixture of experts: softmax router with a choice bias, expert-major row plan, grouped products, weighted combine.
 * ------------------------------------------------------------------------------------------------------------------ */

/* s = softmax(logits[t, 0 : n_experts]); the `top` experts with the largest s + choice_bias (NULL: s; ties: the lower
 * expert) are chosen; weights[t, k] = s[chosen k] / (sum of the chosen s + 1e-20) * scale, or with renorm == 0 the chosen
 * scores themselves, s[chosen k] * scale.  logits: float, row stride logit_stride.  weights: float [n_tokens, top],
 * experts: int32 [n_tokens, top], in order of decreasing choice score. */
int hxm_route_softmax_topk(const float* logits, int64_t logit_stride, const float* choice_bias, int64_t n_tokens,
                           int32_t n_experts, int32_t top, float scale, int32_t renorm, float* weights, int32_t* experts,
                           void* stream);

/* Expert-major order of the n = n_tokens * top (token, choice) pairs: seg[e] .. seg[e + 1] are the rows of expert e
 * (int32 [n_experts + 1]); row_of[t * top + k] = the row of pair (t, k); src[row] = t.  One launch of one workgroup. */
int hxm_moe_plan(const int32_t* experts, int64_t n_tokens, int32_t top, int32_t n_experts, int32_t* seg, int32_t* row_of,
                 int32_t* src, void* stream);

/* Y[r, :] = act(X[src ? src[r] : r, :] . W[e]^T) for the rows r of every expert e (seg as above, n_rows = seg[n_experts]
 * is NOT read by the host: max_rows bounds it).  X: dtype rows of k_dim with stride x_stride; W: dtype [n_experts, n_dim,
 * k_dim]; Y: dtype [max_rows, n_dim].  act: 0 none, 1 squared ReLU.  Products accumulate in float. */
int hxm_grouped_linear(void* y, const void* x, int64_t x_stride, const int32_t* src, const void* w, const int32_t* seg,
                       int64_t max_rows, int32_t n_experts, int64_t n_dim, int64_t k_dim, int32_t act, int dtype, void* stream);

/* out[t, :] = sum_k weights[t, k] * y[row_of[t * top + k], :] + (shared ? sigmoid(shared_gate[t * gate_stride]) * shared[t, :] : 0).
 * A choice whose row_of is negative (an expert beyond the n_experts hxm_moe_plan was called with) adds nothing — or, with
 * `identity` (dtype rows of `width`, row stride identity_stride: the experts' input), weights[t, k] * identity[t, :]: experts
 * without tensors that hand their input on.  y, shared, out: dtype rows of `width`; weights, shared_gate: float. */
int hxm_moe_combine(void* out, const void* y, const int32_t* row_of, const float* weights, const void* shared,
                    const float* shared_gate, int64_t gate_stride, const void* identity, int64_t identity_stride,
                    int64_t n_tokens, int32_t top, int64_t width, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Gated linear recurrence with a matrix state per head (HGRN2): f = low + (1 - low) * sigmoid(f_pre + f_bias) per head and
 * key channel, S <- diag(f) S + (1 - f) v^T, o = S^T silu(q_pre), then o / sqrt(mean(o^2) + eps) * norm_w over each
 * head's value channels.  Gates, state and sums are float.
 * q_pre, f_pre: dtype [n_tokens, heads * dim], v: dtype [n_tokens, heads * vdim] (row strides given); f_bias, low: float
 * [heads * dim]; norm_w: float [vdim]; out: dtype [n_tokens, heads * vdim] contiguous.
 * state: float, slot s at state + s * slot_stride, [heads, dim, vdim] contiguous within a slot.  A sequence whose portion
 * starts at position 0 starts from a zero state (the slot is not read); the slot receives the state after the portion's
 * last token.  q_cu: int32 [n_seq + 1]; positions: int32 [n_tokens]; slots: int32 [n_seq].  ws: float workspace of at least
 * hxm_gated_recurrence_workspace(n_tokens, heads, dim, vdim) floats (the partial results of the key channels' parts).
 * max_q_len: the longest portion of the batch if the caller knows it, else 0; 1 (every sequence brings one token) takes a
 * kernel without the chunk machinery. */
int64_t hxm_gated_recurrence_workspace(int64_t n_tokens, int32_t heads, int32_t dim, int32_t vdim);
int hxm_gated_recurrence(void* out, const void* q_pre, int64_t q_stride, const void* f_pre, int64_t f_stride, const void* v,
                         int64_t v_stride, const float* f_bias, const float* low, const float* norm_w, float eps,
                         float* state, int64_t slot_stride, const int32_t* q_cu, const int32_t* positions,
                         const int32_t* slots, int32_t n_seq, int64_t n_tokens, int32_t heads, int32_t dim, int32_t vdim,
                         int32_t max_q_len, float* ws, int64_t ws_floats, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Grouped-query attention over a paged key/value cache with a linear distance bias and a mask.
 * ------------------------------------------------------------------------------------------------------------------ */

/* From a token's projection row: q = rms_norm(proj[q_off : q_off + q_size]) * q_w -> q_out [n_tokens, q_size] (one norm
 * over the whole query projection, all heads at once; q_w NULL: no norm, a plain copy); when k_size > 0: k likewise with
 * k_w -> the key cache, v (v_size, no norm) -> the value cache, at slot_ids[token] (slot = block * block_size + row; < 0:
 * skipped).  A cache row holds kv_heads heads of head_stride elements; keys fill the first k_size / kv_heads of each,
 * values the first v_size / kv_heads. */
int hxm_qk_norm_cache(const void* proj, int64_t proj_stride, int64_t q_off, int64_t q_size, int64_t k_off, int64_t k_size,
                      int64_t v_off, int64_t v_size, const float* q_w, const float* k_w, float eps, void* q_out,
                      const int32_t* slot_ids, void* key_cache, void* value_cache, int64_t cache_row_stride,
                      int64_t head_stride, int32_t kv_heads, int64_t n_tokens, int dtype, void* stream);

#define HXM_MASK_CAUSAL 0   /* every j <= i */
#define HXM_MASK_WINDOW 1   /* 0 <= i - j < mask_size */
#define HXM_MASK_CHUNK 2    /* j <= i and floor(i / mask_size) == floor(j / mask_size), chunks counted from position 0 */

typedef struct hxm_biased_attn_args {
  void* out;                 /* dtype [n_tokens, n_heads, vdim] contiguous */
  const void* q;             /* dtype [n_tokens, n_heads, dim] contiguous */
  const void* key_cache;     /* dtype paged: block b at + b * cache_block_stride, row r + r * cache_row_stride, head g + g * head_stride */
  const void* value_cache;
  const float* slopes;       /* [n_heads] or NULL: score = q . k * scale - slopes[h] * (i - j) */
  const int32_t* tok_seq;    /* [n_tokens] */
  const int32_t* positions;  /* [n_tokens] */
  const int32_t* block_table;/* flat */
  const int32_t* cu_block_lens; /* [n_seq + 1] */
  int64_t cache_block_stride, cache_row_stride, head_stride;
  int32_t n_tokens, n_heads, kv_heads, dim, vdim, block_size;
  int32_t mask_kind, mask_size;
  float scale;
  int32_t dtype;
  const int32_t* q_cu;       /* [n_seq + 1]: the tile form's portions */
  int32_t n_seq, max_q_len;  /* max_q_len: the longest portion of the batch (1: every sequence decodes) */
  int32_t form;              /* 0: the MFMA forms where they apply (bfloat16, sizes and strides multiples of 8), 1: the row form,
                                2: the MFMA tile form also where the group form (four row tiles sharing each chunk) would run */
  int32_t n_splits;          /* tile form, > 1: a tile's keys are dealt to n_splits waves (<= 64) and merged by a second kernel */
  float* ws_o;               /* n_splits > 1: n_seq * kv_heads * ceil(max_q_len * heads / kv_heads / 16) * n_splits * 16 * ceil16(vdim) floats */
  float* ws_ml;              /* n_splits > 1: ... * n_splits * 32 floats */
  float softcap;             /* > 0: q . k * scale becomes softcap * tanh(q . k * scale / softcap) before the bias; 0: none */
  const float* head_scale;   /* [n_heads] or NULL: head h's scores are q . k * scale * head_scale[h] (a temperature per head) */
  const float* sinks;        /* [n_heads] or NULL: the softmax's denominator of head h holds one more term exp(sinks[h]), which
                                has no key and no value (an attention sink); it is not scaled */
} hxm_biased_attn_args;

/* Softmax attention of every query over the keys of its own sequence that its mask lets it see (scores and weights in
 * float).  Queries of portions and single decoded tokens may share a batch. */
int hxm_biased_attention(const hxm_biased_attn_args* args, void* stream);


/* ------------------------------------------------------------------------------------------------------------------
 * Sequence mixers with per-sequence state beside the paged cache (csrc/seq_ops.hip, csrc/state_scan.hip): short causal
 * convolutions, token shift with several mixes, per-head norm + rotary positions + cache append, decays and step sizes
 * of recurrences, a scan over a matrix state per head (decayed sum, read-before-write with a bonus, delta rule), and the
 * gate / group norm that finishes a mixer.  A sequence's state lives in its state slot: `state` points at the piece's
 * first float in slot 0, slot s is slot_stride floats further.  A portion whose first position is 0 starts from zeros
 * without reading its slot.  q_cu [n_seq + 1]: the batch's portions; positions [n_tokens]; slots [n_seq].
 * ------------------------------------------------------------------------------------------------------------------ */

#define HXM_ACT_NONE 0
#define HXM_ACT_SILU 1
#define HXM_ACT_SIGMOID 2
#define HXM_ACT_TANH 3

/* y[t, c] = act(sum_j w[c, j] u[t - taps + 1 + j, c] + bias[c]) over each sequence, zeros before position 0; the inputs
 * of the taps - 1 positions before a portion come from the slot ([taps - 1, channels] floats, oldest first), which is
 * then brought up to date.  u, y: dtype rows; w: float [channels, taps]; bias: float [channels] or NULL. */
int hxm_causal_conv(void* y, int64_t y_stride, const void* u, int64_t u_stride, const float* w, const float* bias, int act,
                    float* state, int64_t slot_stride, const int32_t* slots, const int32_t* tok_seq, const int32_t* q_cu,
                    const int32_t* positions, int64_t n_tokens, int32_t n_seq, int32_t channels, int32_t taps, int dtype,
                    void* stream);

/* Up to two convolutions of the same inputs in one pass (an input is read once, and the slot brought up to date once):
 * y = act(conv_w(u) + bias) + (skip ? u : 0), and, when y2 is given, y2 = act(conv_w2(u) + bias2) + (skip ? u : 0).  A mixer
 * and a feed-forward that read the same normed input, each through a short convolution of its own added to that input,
 * are one call with skip = 1. */
int hxm_causal_conv_pair(void* y, int64_t y_stride, void* y2, int64_t y2_stride, const void* u, int64_t u_stride, const float* w,
                         const float* w2, const float* bias, const float* bias2, int act, int skip, float* state,
                         int64_t slot_stride, const int32_t* slots, const int32_t* tok_seq, const int32_t* q_cu,
                         const int32_t* positions, int64_t n_tokens, int32_t n_seq, int32_t channels, int32_t taps, int dtype,
                         void* stream);

/* out[m, t, :] = h[t] + (h[t - 1] - h[t]) * mu[m] for m < n_mix, h[t - 1] of the same sequence (zeros before position 0;
 * across portions through the slot's `width` floats, left holding the portion's last h).  h: dtype [n_tokens, width]
 * rows; mu: float [n_mix, width]; out: dtype [n_mix, n_tokens, width] contiguous. */
int hxm_token_shift_mix(void* out, const void* h, int64_t h_stride, const float* mu, int32_t n_mix, float* state,
                        int64_t slot_stride, const int32_t* slots, const int32_t* tok_seq, const int32_t* q_cu,
                        const int32_t* positions, int64_t n_tokens, int32_t n_seq, int64_t width, int dtype, void* stream);

/* y = g * sigmoid(alpha * g) * (u + up_shift) with g = min(gate, limit), u = clamp(up, -limit, limit) (limit <= 0: no
 * clamp).  gate, up: dtype rows (two halves of one projection will do); y: dtype [rows, n]. */
int hxm_clamped_glu(void* y, int64_t y_stride, const void* gate, int64_t gate_stride, const void* up, int64_t up_stride,
                    float limit, float alpha, float up_shift, int64_t rows, int64_t n, int dtype, void* stream);

/* out = act(x) element by element (HXM_ACT_*), dtype rows. */
int hxm_unary(void* out, int64_t out_stride, const void* x, int64_t x_stride, int act, int64_t rows, int64_t n, int dtype,
              void* stream);

/* Per token and head, in float: step = softplus(a[t, h] + step_bias[h]), decay = exp(-exp(log_rate[h]) * step),
 * beta = sigmoid(b[t, h]).  a, b: dtype rows (b NULL: no beta); decay, step, beta: float [n_tokens, heads] (step / beta
 * NULL: not wanted). */
int hxm_head_gates(float* decay, float* step, float* beta, const void* a, int64_t a_stride, const void* b, int64_t b_stride,
                   const float* log_rate, const float* step_bias, int64_t n_tokens, int32_t heads, int dtype, void* stream);

/* decay[t, c] = exp(-exp(x[t, c] + bias[c])) in float.  x: dtype rows; bias: float [n] or NULL; decay: float [rows, n]. */
int hxm_decay_exp(float* decay, const void* x, int64_t x_stride, const float* bias, int64_t rows, int64_t n, int dtype,
                  void* stream);

/* out[t, h, :] = x[t, h, :] / sqrt(sum(x[t, h, :]^2) + eps) * scale in float.  x: dtype rows of heads * dim; out: float
 * [n_tokens, heads * dim]. */
int hxm_unit_norm(float* out, const void* x, int64_t x_stride, float eps, float scale, int64_t n_tokens, int32_t heads,
                  int32_t dim, int dtype, void* stream);

typedef struct hxm_head_rope_args {
  void* q_out;               /* dtype [n_tokens, q_heads * dim] contiguous */
  const void* q;             /* dtype rows of q_heads * dim */
  const void* k;             /* dtype rows of kv_heads * dim */
  int64_t q_stride, k_stride;
  const float* q_w;          /* [dim]: weight of the per-head RMS norm, shared by the heads */
  const float* k_w;
  const float* inv_freq;     /* [rot_dims / 2]: angle of pair i at position p = p * inv_freq[i]; channel i turns with i + rot_dims / 2 */
  const int32_t* positions;  /* [n_tokens] */
  const int32_t* slot_ids;   /* [n_tokens]: cache row of every token (block * block_size + row) */
  void* key_cache;           /* normed and turned keys go here, */
  void* value_cache;         /* the keys as they came (before norm and rotation) here: the layer's values */
  int64_t cache_row_stride, head_stride;
  int64_t n_tokens;
  int32_t q_heads, kv_heads, dim, rot_dims;
  float eps, cos_sin_scale;  /* cos and sin are multiplied by cos_sin_scale */
  int32_t dtype;
} hxm_head_rope_args;

/* Per-head RMS norm (plain weight) of queries and keys, rotary positions on the first rot_dims channels of every head
 * (angles, cos and sin in float), keys and values appended to the paged cache. */
int hxm_head_norm_rope_cache(const hxm_head_rope_args* args, void* stream);

#define HXM_ROT_HALVES 0        /* channel i turns with channel i + dims / 2 */
#define HXM_ROT_INTERLEAVED 1   /* channel 2 i turns with channel 2 i + 1 */
#define HXM_GATE_PER_HEAD 1     /* gate: one number per head, rows of `heads` */
#define HXM_GATE_PER_ELEMENT 2  /* gate: one number per element, rows of heads * size */
#define HXM_ROT_MAX_PARTS 3

typedef struct hxm_rotary_part {
  const void* src;           /* dtype rows: head h of token t at src + t * src_stride + h * src_head_stride, `size` elements */
  void* dst;                 /* dtype rows (dst_stride a token), or the paged cache when to_cache: the token's row is at
                                dst + block * cache_block_stride + row * dst_stride, (block, row) from its slot id */
  const double* inv_freq;    /* [rot_dims / 2]: pair i turns by position * inv_freq[i]; NULL: nothing turns (a copy, or a gate) */
  const void* gate;          /* dtype, optional: the result is multiplied by sigmoid(gate), rows of gate_stride a token */
  int64_t src_stride, src_head_stride, dst_stride, dst_head_stride, cache_block_stride, gate_stride;
  int32_t heads, size;       /* heads of the part, elements of a head */
  int32_t rot_off, rot_dims; /* channels rot_off .. rot_off + rot_dims - 1 of every head turn, the others are copied */
  int32_t layout;            /* HXM_ROT_* */
  int32_t to_cache;
  int32_t gate_kind;         /* HXM_GATE_* */
  float mag;                 /* cos and sin are multiplied by mag */
  float sign;                /* 1: turn by + position; -1: turn back */
} hxm_rotary_part;

typedef struct hxm_rotary_args {
  hxm_rotary_part parts[HXM_ROT_MAX_PARTS];
  const int32_t* positions;  /* [n_tokens] */
  const int32_t* slot_ids;   /* [n_tokens] cache slot (block * block_size + row) of every token; < 0: the token's cache parts are skipped */
  int64_t n_tokens;
  int32_t n_parts, block_size, dtype;
} hxm_rotary_args;

/* Rotary positions over up to three groups of heads of every token in one launch (angles and their cos / sin from the
 * position in double); see hxm_rotary_part.  A part may be turned in place (dst == src with equal strides). */
int hxm_rotary_parts(const hxm_rotary_args* args, void* stream);

#define HXM_SCAN_DECAY 0      /* S <- a S + k (s v)^T;  o = S^T q */
#define HXM_SCAN_BONUS 1      /* o = (S + diag(u) k v^T)^T q;  then S <- a S + k v^T */
#define HXM_SCAN_DELTA 2      /* S <- a S;  S <- S + k (b (v - S^T k))^T;  o = S^T q */

typedef struct hxm_state_scan_args {
  float* out;                /* float [n_tokens, heads * vdim] contiguous */
  const void* q;             /* rows of qk_heads * dim; head h reads q / k head h / (heads / qk_heads) */
  const void* k;
  const void* v;             /* rows of heads * vdim */
  int64_t q_stride, k_stride, v_stride;
  int32_t q_dtype, k_dtype, v_dtype;     /* HX_F32 or HX_BF16, each operand its own */
  int32_t decay_per_channel; /* 0: decay float [n_tokens, heads]; 1: float [n_tokens, heads * dim] (a: one per key channel) */
  const float* decay;
  const float* vscale;       /* float [n_tokens, heads] or NULL: s above (HXM_SCAN_DECAY) */
  const float* beta;         /* float [n_tokens, heads]: b above (HXM_SCAN_DELTA) */
  const float* bonus;        /* float [heads * dim]: u above (HXM_SCAN_BONUS) */
  float* state;              /* the piece [heads, dim, vdim] of every slot */
  int64_t slot_stride;
  const int32_t* slots;
  const int32_t* q_cu;
  const int32_t* positions;
  int64_t n_tokens;
  int32_t n_seq, heads, qk_heads, dim, vdim, mode;
} hxm_state_scan_args;

/* The recurrence of one matrix state S [dim, vdim] per head and sequence, token by token in float, continued from and
 * left in the sequence's slot.  dim <= 256. */
int hxm_state_scan(const hxm_state_scan_args* args, void* stream);

typedef struct hxm_group_norm_args {
  void* out;                 /* dtype rows of n */
  int64_t out_stride;
  const void* x;             /* x_dtype rows of n */
  int64_t x_stride;
  int32_t x_dtype;
  const void* skip;          /* dtype rows of n or NULL: x += skip_w[c / skip_group] * skip */
  int64_t skip_stride;
  const float* skip_w;
  int32_t skip_group;
  const void* gate;          /* dtype rows of n or NULL */
  int64_t gate_stride;
  int32_t gate_act;          /* HXM_ACT_* */
  int32_t gate_first;        /* 1: x *= act(gate) before the norm; 0: after it */
  int32_t group;             /* > 0: every `group` consecutive elements are divided by their root mean square; 0: no norm */
  float eps;
  const float* w;            /* float [w_len] or NULL: element c is multiplied by w[c % w_len] after the norm */
  int32_t w_len;
  float scale;               /* the result is multiplied by scale */
  int64_t rows, n;
  int32_t dtype;
} hxm_group_norm_args;

/* What finishes a mixer: out = scale * [act(gate)] * w * rms_div_groups(x + skip_w * skip [* act(gate)]), in float. */
int hxm_gated_group_norm(const hxm_group_norm_args* args, void* stream);


#ifdef __cplusplus
}
#endif
#endif
