/* C-ABI of libgbx_mixers.so: kernels of sequence mixers, routed feed-forwards and stream updates over RAGGED step batches
 * (gfx950).  A step's rows lie back to back; two int32 tables describe them:
 *   seq [B][4] = slot, position of the sequence's first new row, number of new rows, index of its first row in the step
 *   tok [T][2] = sequence of the step the row belongs to, position of the row
 * dtype codes: 1 = bf16, 2 = fp32 (activation dtype `act`; statistics, scores, gates and the stream are fp32 in both).
 * Every function returns 0 or an error code (1 invalid argument, 2 HIP error, 3 unsupported shape: the caller picks another
 * kernel) and leaves a text for gbxm_last_error().  All launches go to `stream`; nothing synchronises. */
#pragma once
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define GBXM_OK 0
#define GBXM_ERR_INVALID 1
#define GBXM_ERR_HIP 2
#define GBXM_ERR_UNSUPPORTED 3
#define GBXM_BF16 1
#define GBXM_F32 2

int gbxm_version(void);
const char* gbxm_last_error(void);

/* x[t] = table[token[t]] * scale (fp32 stream) and its image h in the activation dtype (h may be null: no image is written). */
int gbxm_embed_scaled(const void* table, const int64_t* tokens, float* x, void* h, int64_t T, int32_t width, float scale,
                      int32_t act, void* stream);
/* In place: rows[t][0:n0] and rows[t][n0:n0+n1] each RMS-normalised over the whole segment (fp32 statistics), times w0 / w1. */
int gbxm_segment_rmsnorm(void* rows, int64_t T, int64_t row_stride, int32_t n0, int32_t n1, const float* w0, const float* w1,
                         float eps, int32_t act, void* stream);
/* x[t] += mult * rms_norm(z[t]) * w, z = branch[t] (top == 1, mix null) or sum_s mix[t][s] * branch[t][s]; h = image of x. */
int gbxm_residual_norm_add(float* x, const void* branch, const float* mix, const float* w, void* h, int64_t T, int32_t width,
                           int32_t top, float eps, float mult, int32_t act, void* stream);
/* out[t] = rms_norm(x[t]) * w in the activation dtype. */
int gbxm_stream_rmsnorm(const float* x, const float* w, void* out, int64_t T, int32_t width, float eps, int32_t act, void* stream);
/* Router decisions from fp32 logits [T][E] (a plain matrix product, left to the vendor library): probabilities over all E, the
 * `top` largest (ties: lower index); weights are the probabilities, divided by their sum if renorm. */
int gbxm_route_topk(const float* logits, int32_t* idx, float* weight, int64_t T, int32_t E, int32_t top, int32_t renorm, void* stream);
/* y[t][s] = down[e] (silu(gate[e] h[t]) * (up[e] h[t])), e = idx[t][s]; gate_up [E][2F][K] (gate rows, then up rows),
 * down [E][K][F].  `ws`: gbxm_expert_glu_workspace bytes (hidden rows; for prompt-sized bf16 steps also the expert-sorted order of
 * the grouped matrix-core products -- gbxm_expert_glu_grouped tells which of the two a call takes). */
size_t gbxm_expert_glu_workspace(int64_t T, int32_t K, int32_t F, int32_t E, int32_t top, int32_t act);
int gbxm_expert_glu_grouped(int64_t T, int32_t K, int32_t F, int32_t E, int32_t top, int32_t act);
int gbxm_expert_glu(const void* h, const void* gate_up, const void* down, const int32_t* idx, void* y, int64_t T, int32_t K,
                    int32_t F, int32_t E, int32_t top, int32_t act, void* ws, size_t ws_bytes, void* stream);

/* Gated sliding-window attention (see gbx-lm_amd/models/window_attention.py for the equations).  qkv rows: q (H*dk) | k (G*dk) |
 * v (G*dv), already normalised; ring caches [slots][window][G*dk] and [slots][window][G*dv] hold positions BEFORE the step. */
typedef struct {
  const void* qkv;
  int64_t row_stride;           /* elements */
  const void* kcache;
  const void* vcache;
  const int32_t* seq;           /* [B][4] */
  const int32_t* tok;           /* [T][2] */
  const int32_t* tiles;         /* [n_tiles][2]: sequence of the step, first row of the tile inside it (prompt kernel) */
  void* out;                    /* [T][H*dv] */
  const float* dist_mul;        /* [H] */
  const float* dist_rate;       /* [H] */
  const float* gate_bias;       /* [H] */
  int64_t T;
  int32_t B, n_tiles, q_tile;
  int32_t H, G, dk, dv, window;
  float scale, softcap;
  int32_t decode_only;          /* every sequence brings one row */
  int32_t act;
  void* partial;                /* optional fp32 [partial_splits][T][H*dv]: lets a step of few rows split its keys over workgroups */
  int32_t partial_splits;
} gbxm_window_attn_args;
int gbxm_window_attention(const gbxm_window_attn_args* a, void* stream);
/* 1 if a step of this kind runs on the matrix-core tile kernel, 0 if on the row kernel (tests and benchmarks name the kernel). */
int gbxm_window_attention_tiled(int32_t dk, int32_t dv, int32_t act, int32_t decode_only);
/* Append the step's k / v rows to the rings (only the last `window` rows of a sequence are written). */
int gbxm_window_append(const void* qkv, int64_t row_stride, int32_t nq, int32_t nk, int32_t nv, void* kcache, void* vcache,
                       const int32_t* seq, const int32_t* tok, int64_t T, int32_t window, int32_t act, void* stream);

/* ---- softmax attention with a sink, rotations, parallel-layer stream update (gbx-lm_amd/models/sink_attention.py) ---- */

/* x[i] += a[i] (+ b[i]) in fp32 over n elements; a, b in the activation dtype (b may be null). */
int gbxm_stream_add(float* x, const void* a, const void* b, int64_t n, int32_t act, void* stream);
/* The same update of rows [T][width], then h[t] = rms_norm(x[t]) * w in the activation dtype (the next layer's input). */
int gbxm_stream_add_norm(float* x, const void* a, const void* b, const float* w, void* h, int64_t T, int32_t width, float eps, int32_t act,
                         void* stream);
/* A matrix per head on few rows: out[t][h][j] = sum_i in[t][h][i] w[h][i][j] (j < n_out), then n_tail channels copied from
 * in[t][h][n_in ..] to out[t][h][n_out ..].  Strides in elements; w is [H][n_in][n_out]. */
int gbxm_head_project(const void* in, int64_t in_row, int64_t in_head, const void* w, void* out, int64_t out_row, int64_t out_head, int64_t T,
                      int32_t H, int32_t n_in, int32_t n_out, int32_t n_tail, int32_t act, void* stream);
/* In place on n elements, fp32 arithmetic: kind 1 = relu(z)^2, 2 = gelu in its tanh form. */
#define GBXM_ACT_RELU2 1
#define GBXM_ACT_GELU_TANH 2
int gbxm_activate(void* z, int64_t n, int32_t kind, int32_t act, void* stream);

/* A run of `heads` heads of `head_dim` channels at `offset` of every row.  Channels [rot_offset, rot_offset + rot_dims) of each head
 * turn by sign * position * freq[i] (pairs i, i + rot_dims/2; or 2i, 2i+1 when interleaved), cos and sin times mult; then the head
 * is scaled to unit root mean square (norm 1) or RMS-normalised with `weight` [head_dim] (norm 2); norm 3 / 4: the same two norms
 * BEFORE the rotation.  All in fp32, in place. */
typedef struct {
  int32_t offset, heads, head_dim, rot_offset, rot_dims, interleaved, norm;
  float mult, sign;
  const float* freq;            /* [rot_dims / 2] */
  const float* weight;          /* [head_dim] for norm 2 */
} gbxm_head_segment;
#define GBXM_MAX_SEGMENTS 4
int gbxm_rotate_norm_heads(void* rows, int64_t T, int64_t row_stride, const int32_t* positions, int64_t pos_stride,
                           const gbxm_head_segment* segs, int32_t n_segs, float eps, int32_t act, void* stream);

/* Slot tables [slots][keep + ring][width]: position p of a sequence lives in row p (p < keep) or keep + (p - keep) % ring.
 * Appends the step's rows (key rows, and value rows unless v is null); of two rows of a step that share a place the later stays. */
int gbxm_slot_append(const void* k, int64_t k_stride, int32_t k_width, const void* v, int64_t v_stride, int32_t v_width, void* kcache,
                     void* vcache, const int32_t* seq, const int32_t* tok, int64_t T, int32_t keep, int32_t ring, int32_t act, void* stream);

/* out[t][h] = gate * sum_j p_j v_j,  p_j = exp(s_j) / (exp(sink_h) + sum_j exp(s_j)),  s_j = scale <q[t][h], k_j> over the keys
 * j <= i of the row's sequence with i - j < window or j < keep.  Keys before the step's first row come from the slot tables, the
 * step's own from k_new / v_new.  Strides in elements; the channel stride is 1 everywhere. */
typedef struct {
  const void* q;      int64_t q_row, q_head;          /* [T][H] x dk */
  const void* k_new;  int64_t k_row, k_head;          /* [T][G] x dk */
  const void* v_new;  int64_t v_row, v_head;          /* [T][G] x dv */
  const void* kcache; int64_t kc_slot, kc_row, kc_head;   /* null when no sequence of the step has history */
  const void* vcache; int64_t vc_slot, vc_row, vc_head;
  const int32_t* seq;           /* [B][4] */
  const int32_t* tok;           /* [T][2] */
  const int32_t* tiles;         /* [n_tiles][2] (prompt kernel) */
  void* out;                    /* [T][H*dv] */
  const float* sink;            /* [H], or null: plain softmax */
  const void* gate;  int64_t gate_row;                /* [T][H] activation dtype, or null: out *= sigmoid(gate) */
  int64_t T;
  int32_t B, n_tiles, q_tile;
  int32_t H, G, dk, dv;
  int32_t window;               /* <= 0: every earlier key is seen */
  int32_t keep, ring;
  float scale;
  int32_t decode_only, act;
  void* partial;                /* optional fp32 [partial_splits][T][H][(dv + 3) / 4 * 4 + 4] */
  int32_t partial_splits;
} gbxm_sink_attn_args;
int gbxm_sink_attention(const gbxm_sink_attn_args* a, void* stream);
int gbxm_sink_attention_tiled(int32_t dk, int32_t dv, int32_t act, int32_t decode_only);

/* ---- several residual streams, layer norm, gated activations, grouped sigmoid router (gbx-lm_amd/models/residual.py:hyper_step_,
 * models/feed_forward.py:glu_, models/switch_layers.py) ---- */

/* One sublayer boundary over streams X fp32 [T][S][width], in place, one workgroup per row:
 *   if y:  z = y[t] (top == 1) or sum_k y_mix[t][k] y[t][k];   X_j <- sum_i mix[i][j] X_i + write[j] z   (all j from the old X)
 *   u = sum_i read[i] X_i   (read null: plain sum)
 *   norm_w: h = (u - mean) / sqrt(var + eps) * norm_w + norm_b in the activation dtype (var = mean of squared deviations), else
 *   out_u = u (fp32).  S <= 8. */
int gbxm_hyper_step(float* X, const void* y, const float* y_mix, const float* mix, const float* write, const float* read, const float* norm_w,
                    const float* norm_b, void* h, float* out_u, int64_t T, int32_t S, int32_t width, int32_t top, float eps, int32_t act,
                    void* stream);
/* out[t][f] = act(gu[t][f], gu[t][F + f]) in fp32, rows of 2F in, F out (unit inner strides, row strides in elements).
 * kind 1: g sigmoid(g) u;  kind 2: g' = min(g, limit), u' = clamp(u, -limit, limit), g' sigmoid(alpha g') (u' + 1). */
#define GBXM_GLU_SILU 1
#define GBXM_GLU_CLAMPED_SWISH 2
#define GBXM_GLU_GELU_TANH 3      /* gelu(g) u, gelu in its tanh form */
#define GBXM_GLU_SIGMOID 4        /* sigmoid(g) u */
int gbxm_glu(const void* gu, int64_t gu_stride, void* out, int64_t T, int32_t F, int32_t kind, float limit, float alpha, int32_t act, void* stream);
/* Router decisions from fp32 logits [T][E]: s = sigmoid(logit), choice score c = s + correction; with n_groups > 0 the experts form
 * n_groups equal groups of neighbours, a group's score is the sum of its two largest c, and only experts of the keep_groups best
 * groups can be chosen; the `top` largest c are chosen (ties: lower index); weight = s (divided by the chosen sum + 1e-20 if
 * renorm) * scale. */
int gbxm_route_sigmoid_groups(const float* logits, const float* correction, int32_t* idx, float* weight, int64_t T, int32_t E, int32_t top,
                              int32_t n_groups, int32_t keep_groups, int32_t renorm, float scale, void* stream);
/* gbxm_expert_glu with the expert's activation as a parameter (GBXM_GLU_*, alpha = 1.702 for kind 2). */
int gbxm_expert_glu_act(const void* h, const void* gate_up, const void* down, const int32_t* idx, void* y, int64_t T, int32_t K, int32_t F,
                        int32_t E, int32_t top, int32_t act, int32_t kind, float limit, void* ws, size_t ws_bytes, void* stream);

/* ---- recurrent mixers: a decayed matrix state per head (gbx-lm_amd/models/recurrent_mixers.py) ---- */

/* Row preparation, everything in fp32.  y rows hold q (G*dk) | k (G*dk) | v (H*dv) at off_q / off_k / off_v and optionally beta (H) at
 * off_beta (< 0: none); `a` rows [T][H*dk] are the decay projection.  With conv (rows [2 G dk + H dv][taps], q | k | v must be adjacent
 * from off_q on): c[t] = silu(sum_j conv[c][j] in[t - (taps-1) + j]), inputs before the step from tail [slots][taps-1][C] (oldest
 * first), zeros before the sequence.  unit: q, k heads / sqrt(sum sq + 1e-6).  out row: q * q_scale | k | v | decay | beta with
 * decay = exp(-rate[h] * softplus(sign * (a + bias))), beta = sigmoid(.).  `a` null (then decay_bias may be null): decay = rate[h]. */
typedef struct {
  const void* y;    int64_t y_stride;
  const void* a;    int64_t a_stride;
  const void* conv;             /* activation dtype, or null */
  const void* tail;             /* activation dtype [slots][taps-1][C] */
  const float* decay_bias;      /* [H*dk] */
  const float* decay_rate;      /* [H] */
  const int32_t* seq;           /* [B][4] */
  const int32_t* tok;           /* [T][2] */
  float* out;       int64_t out_stride;
  int64_t T;
  int32_t H, G, dk, dv, off_q, off_k, off_v, off_beta, taps, unit;
  float sign, q_scale;
  int32_t act;
  int32_t qkv_silu;             /* without conv: q | k | v pass silu */
} gbxm_recurrent_prep_args;
int gbxm_recurrent_prepare(const gbxm_recurrent_prep_args* a, void* stream);
/* tail[slot] <- the last taps-1 inputs (channels [0, C) of y) of every sequence of the step; older ones shift out. */
int gbxm_conv_tail_update(const void* y, int64_t y_stride, void* tail, const int32_t* seq, int32_t B, int32_t C, int32_t taps, int32_t act,
                          void* stream);
/* The scan over each sequence's new rows.  r: rows of gbxm_recurrent_prepare; state fp32 [slots][H][dv][dk] (read unless the sequence
 * starts at position 0, written back); out fp32 [T][H*dv].  Per token: S <- diag(decay) S; delta: u = beta (v - S^T k) else u = v;
 * S <- S + k u^T; o = S^T q.  T: rows of the step (chooses the workgroup shape).  dk <= 256. */
int gbxm_state_scan(const float* r, int64_t r_stride, float* state, float* out, const int32_t* seq, int32_t B, int64_t T, int32_t H, int32_t G,
                    int32_t dk, int32_t dv, int32_t delta, void* stream);
/* out[t][h][c] = o[t][h][c] / sqrt(mean_c o^2 + eps) * w[c] * gate(g[t][h][c]); gate kind 1 silu, 2 sigmoid; o fp32, g / out activation dtype. */
int gbxm_head_norm_gate(const float* o, const void* gate, int64_t gate_stride, const float* w, void* out, int64_t T, int32_t H, int32_t dv,
                        float eps, int32_t kind, int32_t act, void* stream);

/* ---- sandwich-norm layers, token shift, hashed pair embedding (gbx-lm_amd/models/residual.py, models/embedding.py) ---- */

/* x[t] = table[token[t]] + pair[row], row = (prev * mul_prev + token * mul_cur) mod buckets, or `buckets` for a sequence's first token;
 * prev = the row before in the step, or state[slot] (int64) for the step's first row.  state[slot] <- the sequence's last token. */
int gbxm_embed_hashed_pair(const void* table, const void* pair, const int64_t* tokens, int64_t* state, const int32_t* seq, const int32_t* tok,
                           float* x, int64_t T, int32_t width, int64_t buckets, int64_t mul_prev, int64_t mul_cur, int32_t act, void* stream);
/* n[t] = rms_norm(x[t]) * w;  h[t] = n[t] + (n[t-1] - n[t]) * shift in the activation dtype; n[t-1] of a step's first row is
 * state[slot] (fp32 [slots][width]) or zero at position 0; state[slot] <- n of the sequence's last row. */
int gbxm_norm_token_shift(const float* x, const float* w, const float* shift, float* state, const int32_t* seq, const int32_t* tok, void* h,
                          int64_t T, int32_t width, float eps, int32_t act, void* stream);
/* z = branch[t] (top == 1) or sum_k mix[t][k] branch[t][k], plus extra[t] if given;  x[t] += rms_norm(z) * w;  with next_w:
 * h[t] = rms_norm(x[t]) * next_w in the activation dtype. */
int gbxm_branch_norm_add_norm(float* x, const void* branch, const float* mix, const void* extra, const float* w, const float* next_w, void* h,
                              int64_t T, int32_t width, int32_t top, float eps, int32_t act, void* stream);
/* out[t] = (rms_norm(a[t]) * wa + rms_norm(b[t]) * wb) / 2, rows of the activation dtype. */
int gbxm_normed_pair_mean(const void* a, const void* b, const float* wa, const float* wb, void* out, int64_t T, int32_t width, float eps,
                          int32_t act, void* stream);
/* out[t][f] = act(gate[t][f]) * up[t][f] (GBXM_GLU_SILU / GELU_TANH / SIGMOID), row strides in elements, out rows contiguous. */
int gbxm_gate_mul(const void* gate, int64_t gate_stride, const void* up, int64_t up_stride, void* out, int64_t T, int32_t F, int32_t kind,
                  int32_t act, void* stream);

/* ---- gated linear recurrent unit (gbx-lm_amd/models/gated_lru.py) ---- */

/* out[t][c] = bias[c] + sum_j conv[c][j] x[t - (taps-1) + j][c] in fp32; inputs before the step from tail [slots][taps-1][C] (oldest
 * first; the activation dtype), zeros before the sequence.  bias may be null. */
int gbxm_causal_conv_rows(const void* x, int64_t x_stride, const void* conv, const float* bias, const void* tail, const int32_t* seq,
                          const int32_t* tok, float* out, int64_t T, int32_t C, int32_t taps, int32_t act, void* stream);
/* logits[t][b][o] = bias[b][o] + sum_i w[b][o][i] u[t][b * bs + i], o < n_out; u fp32 [T][blocks * bs], w [blocks][n_out][bs] in the
 * activation dtype, fp32 sums in a fixed order. */
int gbxm_block_gate_logits(const float* u, const void* w, const float* bias, float* logits, int64_t T, int32_t blocks, int32_t bs, int32_t n_out,
                           int32_t act, void* stream);
/* logits: element (t, b, o) at t * lg_t + b * lg_b + o (floats).  Per channel c of block b = c / bs:  r = sigmoid(logits[t][b][c % bs]),
 * i = sigmoid(logits[t][b][bs + c % bs]),
 * a = exp(-rate * r * lam_sp[c]), S <- a S + sqrt(1 - a^2) i u[t][c] over each sequence's rows from state[slot][c] (zero at position
 * 0; written back); out[t][c] = S * gelu_tanh(y[t][c]) in the activation dtype. */
int gbxm_gated_lru_scan(const float* u, const float* logits, int64_t lg_t, int64_t lg_b, const float* lam_sp, const void* y, int64_t y_stride, float* state, void* out,
                        const int32_t* seq, int32_t B, int64_t T, int32_t C, int32_t bs, float rate, int32_t act, void* stream);

#ifdef __cplusplus
}
#endif
