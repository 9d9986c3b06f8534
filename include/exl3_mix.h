/*
 * exl3_mix.h -- C-ABI of the sequence-mixer library (libexl3_mix.so): the kernels of models whose layers are not the
 * quantized-linear transformer block of libexl3_hip.so -- sliding-window attention with a learned sink over a ring cache, gated
 * linear attention with a per-channel decay and a carried state, RMS norms over a 32-bit residual stream, a gated residual,
 * the PolyNorm activation, top-k routers and unquantized experts; latent attention (a low-rank key/value cache with rotary positions), the
 * Dynamic Tanh norm and the residual updates of pre-norm blocks.
 *
 * Conventions (the same as exl3_hip.h): plain device pointers, sizes and scalars; `stream` is a hipStream_t; calls are
 * asynchronous; return 0 on success and < 0 on error with the text in exl3_mix_last_error() (thread-local).
 *
 *   - `dtype` names the element type of activations and of matrix weights: EXL3_MIX_BF16 or EXL3_MIX_F32.  The residual stream,
 *     norm weights, biases read by these kernels, sinks, decay biases, recurrent states, scores and softmax weights are float32
 *     in both modes.
 *   - A step's tokens are PACKED: N rows, the sequences of a batch one behind the other without padding.  cu[b] .. cu[b+1] are the
 *     rows of sequence b; tok_seq[n] / tok_pos[n] give a row's sequence and its position in that sequence (counted from 0 over the
 *     sequence's whole life, not over the step).  slots[b] is the sequence's slot in the state buffers.
 *   - A row stride `*_ld` counts elements between consecutive rows, so that a kernel reads a column block of a wider matrix product
 *     in place.
 */
#ifndef EXL3_MIX_H
#define EXL3_MIX_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EXL3_MIX_OK        0
#define EXL3_MIX_ERR_ARG  (-1)
#define EXL3_MIX_ERR_HIP  (-2)

#define EXL3_MIX_BF16 0
#define EXL3_MIX_F32  1

/* gated activations of two projections g (gate) and u (up):  SILU: silu(g) u;  CLAMPED_SWISH: g' = min(g, limit), u' = clamp(u, -limit, limit),
 * g' sigmoid(1.702 g') (u' + 1). */
#define EXL3_MIX_GLU_SILU          0
#define EXL3_MIX_GLU_CLAMPED_SWISH 1
/* plain activations */
#define EXL3_MIX_ACT_RELU2     0
#define EXL3_MIX_ACT_GELU_TANH 1
#define EXL3_MIX_ACT_SILU      2

/* attention masks: WINDOW: a row sees the last `window` positions up to itself; CHUNK: the positions up to itself inside its own chunk of `window`
 * positions (a chunk starts where the sequence's position is a multiple of `window`). */
#define EXL3_MIX_MASK_WINDOW 0
#define EXL3_MIX_MASK_CHUNK  1

#define EXL3_MIX_ABI_VERSION 4

const char* exl3_mix_last_error(void);
int  exl3_mix_abi_version(void);

/* x[n] = table[tokens[n]] * scale (float32 residual);  if norm_w: h[n] = x[n] / sqrt(mean(x[n]^2) + eps) * norm_w. */
int exl3_mix_embed(float* x, void* h, const void* table, const int32_t* tokens, float scale, const float* norm_w, float eps,
                   int n, int width, int vocab, int dtype, void* stream);

/* h[i] = rms_norm(x[rows ? rows[i] : i]) * w: RMS norm of selected residual rows (the model's last norm runs on the wanted rows only). */
int exl3_mix_rms_norm_rows(void* h, const float* x, const int32_t* rows, const float* w, float eps, int n, int width, int dtype, void* stream);

/* Gated residual: x[n] += y[n] * sigmoid(r[n])  (r holds the gate's pre-activation, bias included), then, if norm_w, the next
 * sublayer's input h[n] = rms_norm(x[n]) * norm_w.  y and r are column blocks of wider matrices (row strides y_ld, r_ld). */
int exl3_mix_gated_residual(float* x, const void* y, int64_t y_ld, const void* r, int64_t r_ld, const float* norm_w, void* h, float eps,
                            int n, int width, int dtype, void* stream);

/* PolyNorm: out = a N(z) + b N(z^2) + c N(z^3) + e with N(u) = u / sqrt(mean(u^2) + eps) over a row; coef = {a, b, c, e} (float32, device). */
int exl3_mix_polynorm(void* out, const void* z, int64_t z_ld, const float* coef, float eps, int n, int ff, int dtype, void* stream);

/* Values of a step enter the attention cache: every key/value head's value is divided by its root mean square (eps inside the
 * root, no weight) and written to v_norm [n][kv_heads][vdim]; keys and normalised values of the rows that are among the last
 * `window` positions of their sequence (tok_pos >= len_after[seq] - window) go to the ring buffers
 * ring_k [slots][window][kv_heads][dim], ring_v [slots][window][kv_heads][vdim] at position tok_pos % window. */
int exl3_mix_attn_store(void* v_norm, void* ring_k, void* ring_v, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                        const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, const int32_t* len_after,
                        float eps, int n, int kv_heads, int dim, int vdim, int window, int dtype, void* stream);

/* Sliding-window attention with a sink over the step's own keys (sequences that start at position 0 in this step):
 * row i sees rows j of its sequence with 0 <= i - j < window; weights = exp(s_j - m) / (exp(sink_h - m) + sum_j exp(s_j - m)),
 * s_j = scale * q.k_j; out[n][h] = sigmoid(gate[n][h]) * sum_j w_j v_j.  sink may be NULL (plain softmax), gate may be NULL.
 * v_norm as written by exl3_mix_attn_store.  Scores, weights and sums are float32. */
int exl3_mix_attn_prefill(void* out, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v_norm,
                          const void* gate, int64_t gate_ld, const float* sink, const int32_t* cu, const int32_t* tok_seq, const int32_t* tok_pos,
                          int n, int heads, int kv_heads, int dim, int vdim, float scale, int window, int dtype, void* stream);

/* The same on the matrix cores, bfloat16 only (scores, maxima, exponentials and sums stay float32; the weights are rounded to bfloat16 for the
 * product with the values): dim, vdim <= 256; `max_rows` = the longest sequence of the step. */
int exl3_mix_attn_prefill_mfma(void* out, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v_norm,
                               const void* gate, int64_t gate_ld, const float* sink, const int32_t* cu,
                               int batch, int max_rows, int heads, int kv_heads, int dim, int vdim, float scale, int window, void* stream);

/* The same for one new row per sequence against the ring buffers (which already hold the row's own key and value):
 * row b sees the min(len_after[b], window) newest entries of slot slots[b]. */
int exl3_mix_attn_decode(void* out, const void* q, int64_t q_ld, const void* ring_k, const void* ring_v,
                         const void* gate, int64_t gate_ld, const float* sink, const int32_t* slots, const int32_t* len_after,
                         int n, int heads, int kv_heads, int dim, int vdim, float scale, int window, int dtype, void* stream);

/* Gated linear attention, token by token (prefill of any length and decode): per sequence b and head h, with the state S [dim][vdim]
 * (float32, state [slots][heads][dim][vdim]; taken as zero where pos0[b] == 0, read from slot slots[b] otherwise, written back at the end):
 *     alpha_t = exp(log_sigmoid(z_t) / tau),  z_t = a2 . lr_t + a2_bias      (lr: the low-rank decay input [n][rank], a2 [heads*dim][rank])
 *     S <- diag(alpha_t) S + k_t v_t^T,   o_t = S^T (q_t * q_scale)
 * o [n][heads][vdim] float32. */
int exl3_mix_gla_scan(float* o, float* state, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                      const void* lr, int64_t lr_ld, const void* a2, const float* a2_bias, const int32_t* cu, const int32_t* slots, const int32_t* pos0,
                      int batch, int heads, int dim, int vdim, int rank, float tau, float q_scale, int dtype, void* stream);

/* The same results (up to float32 rounding) for long prompts, with the time axis cut into `segs` segments of `seg_len` rows per sequence
 * (segs * seg_len >= the longest sequence of the step) that run in parallel: every segment first runs from a zero state and leaves its local
 * state and the product of its decays, a short pass chains these into the state each segment starts from (and the slot's final state), and
 * every segment runs again from there and writes its outputs.  seg_state [batch*segs][heads][dim][vdim], seg_decay [batch*segs][heads][dim]: scratch. */
int exl3_mix_gla_segmented(float* o, float* state, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                           const void* lr, int64_t lr_ld, const void* a2, const float* a2_bias, const int32_t* cu, const int32_t* slots, const int32_t* pos0,
                           int batch, int heads, int dim, int vdim, int rank, float tau, float q_scale, int segs, int seg_len,
                           float* seg_state, float* seg_decay, int dtype, void* stream);

/* out[n][h*vdim + v] = o[n][h][v] / sqrt(mean_v(o[n][h]^2) + eps) * w[v] * silu(g[n][h*vdim + v]) */
int exl3_mix_gla_out(void* out, const float* o, const float* w, const void* g, int64_t g_ld, float eps, int n, int heads, int vdim, int dtype, void* stream);

/* Router: the `top` largest of `experts` logits per row (float32; ties go to the lower index), weights = softmax over the chosen logits. */
int exl3_mix_topk_softmax(int32_t* idx, float* wts, const float* logits, int n, int experts, int top, void* stream);

/* Experts of a few rows, weights streamed once per (row, choice): hid[n*top + r] = silu(Wg[e] h[n]) * (Wu[e] h[n]) with e = idx[n][r];
 * Wg, Wu [experts][ff][width]. */
int exl3_mix_moe_gate_up(void* hid, const void* h, const void* wg, const void* wu, const int32_t* idx, int n, int top, int experts, int ff, int width,
                         int dtype, void* stream);
/* y[n] = sum_r wts[n][r] * Wd[idx[n][r]] hid[n*top + r];  Wd [experts][width][ff]. */
int exl3_mix_moe_down(void* y, const void* hid, const void* wd, const int32_t* idx, const float* wts, int n, int top, int experts, int ff, int width,
                      int dtype, void* stream);

/* Experts of a handful to a few dozen rows, expert-major: every expert's weights are streamed once for all the rows that chose it.
 * hid [n*top][ff] (scratch), per [n*top][width] = the unweighted expert outputs per (row, choice); exl3_mix_moe_combine with where[i] = i adds the
 * choices with their weights.  Rows must be 16-byte aligned multiples of 8 (bfloat16) / 4 (float32) elements. */
int exl3_mix_moe_expert_major(void* per, void* hid, const void* h, const void* wg, const void* wu, const void* wd, const int32_t* idx,
                              int n, int top, int experts, int ff, int width, int dtype, void* stream);

/* Experts of many rows run as vendor matrix products over rows sorted by expert; these two kernels sit between and behind them:
 * out = silu(g) * u element by element, and y[n] = sum_r wts[n][r] * sorted[where[n*top + r]] (rows back in token order, weighted). */
int exl3_mix_silu_mul(void* out, const void* g, const void* u, int64_t count, int dtype, void* stream);
int exl3_mix_moe_combine(void* y, const void* sorted, const int32_t* where, const float* wts, int n, int top, int width, int dtype, void* stream);

/* The same experts with the gated activation named by `act` (EXL3_MIX_GLU_*) and its clamp `limit`. */
int exl3_mix_moe_gate_up_act(void* hid, const void* h, const void* wg, const void* wu, const int32_t* idx, int n, int top, int experts, int ff, int width,
                             int act, float limit, int dtype, void* stream);
int exl3_mix_moe_expert_major_act(void* per, void* hid, const void* h, const void* wg, const void* wu, const void* wd, const int32_t* idx,
                                  int n, int top, int experts, int ff, int width, int act, float limit, int dtype, void* stream);

/* ---- pre-norm blocks whose norm needs no statistics, and the pieces between their matrix products (mix_rowops.hip) ---- */

/* x[n] = table[tokens[n]] (float32 residual); if xc: the same row in the activation type at xc + n * xc_ld. */
int exl3_mix_embed_copy(float* x, void* xc, int64_t xc_ld, const void* table, const int32_t* tokens, int n, int width, int vocab, int dtype, void* stream);

/* Residual update fused with what the next consumer reads.  mode 0: x stays (y unused); 1: x += y'; 2: x = y', where y' = y, or, with rms_w,
 * y / sqrt(mean(y^2) + eps) * rms_w.  out 0: nothing; 1: h = x in the activation type; 2: h = tanh(alpha x) * w + b (Dynamic Tanh: no mean, no
 * variance).  y and h may be column blocks (row strides y_ld, h_ld). */
int exl3_mix_residual_norm(float* x, const void* y, int64_t y_ld, int mode, const float* rms_w, float eps, int out, float alpha, const float* w, const float* b,
                           void* h, int64_t h_ld, int n, int width, int dtype, void* stream);

/* h[i] = tanh(alpha * x[rows ? rows[i] : i]) * w + b: the last norm on the wanted rows only. */
int exl3_mix_dyn_tanh_rows(void* h, const float* x, const int32_t* rows, float alpha, const float* w, const float* b, int n, int width, int dtype, void* stream);

/* out[n][i] = act(z[n][i]) (EXL3_MIX_ACT_*), and out[n][i] = glu(g[n][i], u[n][i]) (EXL3_MIX_GLU_*, `limit` for the clamped kind); out is contiguous. */
int exl3_mix_act(void* out, const void* z, int64_t z_ld, int n, int ff, int kind, int dtype, void* stream);
int exl3_mix_glu_act(void* out, const void* g, int64_t g_ld, const void* u, int64_t u_ld, int n, int ff, int kind, float limit, int dtype, void* stream);

/* out[n][j] = gelu_tanh(gate[n][j]) * table[tokens[n]][col0 + j], j < dim: a gate multiplied with a slice of a per-token embedding row. */
int exl3_mix_token_gate(void* out, const void* gate, int64_t gate_ld, const void* table, int64_t table_ld, int col0, const int32_t* tokens,
                        int n, int dim, int vocab, int dtype, void* stream);

/* out[n][h * vdim + v] = a[n * a_row + h * a_head + v] * (gate ? sigmoid(gate[n][h * vdim + v]) : 1): an element-wise output gate over heads that may lie
 * head-major (the result of a per-head batched product). */
int exl3_mix_heads_gate(void* out, const void* a, int64_t a_row, int64_t a_head, const void* gate, int64_t gate_ld, int n, int heads, int vdim, int dtype, void* stream);

/* Router with independent scores s = sigmoid(z): the `top` experts with the largest s + correction (correction may be NULL; ties go to the lower index);
 * weights = s / (sum of the chosen s + 1e-20) * scale, or s * scale with normalise = 0. */
int exl3_mix_topk_sigmoid(int32_t* idx, float* wts, const float* logits, const float* correction, float scale, int normalise, int n, int experts, int top, void* stream);

/* ---- latent attention (mix_latent.hip): per token one low-rank latent c [rank] and one rotated key part k_rot [rot_dim] shared by all heads ---- */

/* From dkv [n][rank + rot_dim]: c = rms_norm(dkv[:rank]) * norm_w; k_rot = the rest with rotary positions on its first rot_dims entries (interleaved
 * pairs (2i, 2i+1), angle = tok_pos * freq[i], cos and sin times `mag`, all float32).  [c | k_rot] goes to ckr [n][rank + rot_dim] and, for the rows among
 * the last `window` positions of their sequence, to ring [slots][window][rank + rot_dim] at tok_pos % window.  The same rotation is applied in place to
 * the last rot_dim entries of every head of q [n][heads][dim + rot_dim]. */
int exl3_mix_latent_prep(void* ckr, void* ring, const void* dkv, int64_t dkv_ld, const float* norm_w, void* q, int64_t q_ld,
                         const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, const int32_t* len_after,
                         const float* freq, float mag, float eps, int n, int heads, int dim, int rot_dim, int rot_dims, int rank, int window, int dtype, void* stream);

/* k [n][heads][dim + rot_dim]: the last rot_dim entries of every head = k_rot of the row (ckr as written by exl3_mix_latent_prep). */
int exl3_mix_latent_fill_k(void* k, int64_t k_ld, const void* ckr, int n, int heads, int dim, int rot_dim, int rank, int dtype, void* stream);

/* One new row per sequence against the ring in the absorbed form: score_j = scale * (q_lat . c_j + q_rot . k_rot_j) over the min(len_after, window) newest
 * entries, softmax (with exp(sink_h) in the denominator if sink), o_lat = sum_j w_j c_j.  q_lat (the head's unrotated query carried into the latent space)
 * and o_lat are addressed as base + n * row_stride + h * head_stride; q_rot is read from q [n][heads][dim + rot_dim].  rank <= 1024. */
int exl3_mix_latent_decode(void* o_lat, int64_t o_row, int64_t o_head, const void* q_lat, int64_t ql_row, int64_t ql_head, const void* q, int64_t q_ld,
                           const void* ring, const float* sink, const int32_t* slots, const int32_t* len_after,
                           int n, int heads, int dim, int rot_dim, int rank, float scale, int window, int dtype, void* stream);

/* The same on the matrix cores, bfloat16 only: sixteen heads share every read of a cached row; the cached rows of a sequence are split over `splits`
 * workgroups whose partial sums a second kernel merges (the sink enters there).  rank and rot_dim multiples of 8, rank <= 512, rot_dim <= 128.  `scratch`
 * holds exl3_mix_latent_decode_mfma_scratch(...) floats. */
int exl3_mix_latent_decode_mfma_scratch(int n, int heads, int rank, int splits, int64_t* floats);
int exl3_mix_latent_decode_mfma(void* o_lat, int64_t o_row, int64_t o_head, const void* q_lat, int64_t ql_row, int64_t ql_head, const void* q, int64_t q_ld,
                                const void* ring, const float* sink, const int32_t* slots, const int32_t* len_after, float* scratch, int splits,
                                int n, int heads, int dim, int rot_dim, int rank, float scale, int window, void* stream);

/* ---- several attention maps per head, chunk masks, soft-capped scores (mix_attn.hip, mix_attn_mfma.hip, mix_diffattn.hip) ---- */

/* The attention kernels above with: `maps` maps per head (queries [n][heads][maps][dim], keys [.][kv_heads][maps][dim]; every map of a head reads the values
 * of the head's key/value head; out [n][heads][maps][vdim]; a gate needs maps == 1), scores soft-capped to softcap tanh(score / softcap) (softcap 0: none),
 * mask EXL3_MIX_MASK_* over `window` positions, values as a column block (v_ld), and the result in float32 (out_f32) or the activation type.
 * Decode with the chunk mask reads the ring entries 0 .. (len_after - 1) % window. */
int exl3_mix_attn_prefill_ex(void* out, int out_f32, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                             const void* gate, int64_t gate_ld, const float* sink, const int32_t* cu, const int32_t* tok_seq, const int32_t* tok_pos,
                             int n, int heads, int kv_heads, int maps, int dim, int vdim, float scale, float softcap, int window, int mask, int dtype, void* stream);
int exl3_mix_attn_prefill_mfma_ex(void* out, int out_f32, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                                  const void* gate, int64_t gate_ld, const float* sink, const int32_t* cu,
                                  int batch, int max_rows, int heads, int kv_heads, int maps, int dim, int vdim, float scale, float softcap, int window, int mask,
                                  void* stream);
int exl3_mix_attn_decode_ex(void* out, int out_f32, const void* q, int64_t q_ld, const void* ring_k, const void* ring_v,
                            const void* gate, int64_t gate_ld, const float* sink, const int32_t* slots, const int32_t* len_after,
                            int n, int heads, int kv_heads, int maps, int dim, int vdim, float scale, float softcap, int window, int mask, int dtype, void* stream);

/* Differential attention of a prompt step on the matrix cores, bfloat16 only: both maps of a head in one workgroup (the value tile is staged once for both)
 * and the combination in the epilogue: out[n][h] = rms_unit(a1 - lambda a2) (1 - diff) sigmoid(gate[n][h]) (exl3_mix_diff_combine), with a1 / a2 the
 * head's two attention maps (queries [n][heads][2][dim], keys [n][kv_heads][2][dim], values [n][kv_heads][vdim]) kept in float32 registers.
 * dim <= 128, vdim <= 256, scale > 0. */
int exl3_mix_attn_prefill_mfma_diff(void* out, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                                    const void* gate, int64_t gate_ld, const int32_t* cu, int batch, int max_rows, int heads, int kv_heads, int dim, int vdim,
                                    float scale, float softcap, int window, int mask, float lambda, float diff, float eps, void* stream);

/* Queries and keys before the attention core, in place: per (row, head) RMS norm over dim with the weight q_norm / k_norm [dim] (NULL: none), then rotary
 * positions on the first rot_dims entries (freq [rot_dims / 2], NULL: none): pairs (i, i + rot_dims/2), or (2i, 2i+1) when `interleaved`; angle =
 * tok_pos * freq[i], cos and sin times `mag`.  q_heads and k_heads count every (head, map).  Keys and values of the rows with tok_pos >= len_after - window
 * go to ring_k [slots][window][k_heads][dim] and ring_v [slots][window][v_heads][vdim] at tok_pos % window. */
int exl3_mix_qk_prep(void* q, int64_t q_ld, void* k, int64_t k_ld, const void* v, int64_t v_ld, const float* q_norm, const float* k_norm,
                     const float* freq, int rot_dims, float mag, int interleaved, float eps, void* ring_k, void* ring_v,
                     const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, const int32_t* len_after,
                     int n, int q_heads, int k_heads, int v_heads, int dim, int vdim, int window, int dtype, void* stream);

/* Differential attention: a [n][heads][2][vdim] float32 (the two maps of every head);  o = a1 - lambda a2;
 * out[n][h][c] = o_c / sqrt(mean_c(o^2) + eps) * (1 - diff) * sigmoid(gate[n][h])  (gate NULL: no gate). */
int exl3_mix_diff_combine(void* out, const float* a, float lambda, float diff, float eps, const void* gate, int64_t gate_ld,
                          int n, int heads, int vdim, int dtype, void* stream);

/* ---- pre-norm blocks with a short causal input convolution (mix_canon.hip) ---- */

/* Residual update fused with the next RMS norm: mode 0: x stays; 1: x += y; 2: x = y.  If h: hn = x / sqrt(mean(x^2) + eps) * w.  Without conv_w, h = hn.
 * With conv_w [taps][width] (steps of ONE row per sequence): h = hn + sum_j conv_w[j][c] hn_(pos - taps + 1 + j), the earlier rows read from
 * ring [slots][taps - 1][width] (entry = position % (taps - 1); positions below 0 are zero rows), and hn is stored there. */
int exl3_mix_residual_rms(float* x, const void* y, int64_t y_ld, int mode, const float* w, float eps, void* h, int64_t h_ld,
                          const float* conv_w, int taps, void* ring, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots,
                          int n, int width, int dtype, void* stream);

/* The same convolution (conv_w [taps][width]) over a packed step whose sequences start in it (or bring one row each): out = hn + conv(hn), predecessors from the step's own rows
 * where tok_pos - back >= pos0[seq], from the ring otherwise; the rows at the last taps - 1 positions of every sequence are stored in the ring. */
int exl3_mix_canon(void* out, int64_t out_ld, const void* hn, int64_t hn_ld, const float* conv_w, int taps, void* ring,
                   const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, const int32_t* pos0, const int32_t* len_after,
                   int n, int width, int dtype, void* stream);

/* x <- cap * tanh(x / cap) over `count` float32 values in place (soft-capped logits). */
int exl3_mix_softcap(float* x, int64_t count, float cap, void* stream);

/* ---- routers over groups of experts, experts without weights, ungated experts (mix_rowops.hip, mix_moe.hip) ---- */

/* Router over `total` outputs: the first `real` name stored experts, the others experts that return their input.  Scores s: softmax over all outputs
 * (kind 0) or sigmoids (kind 1); the choice looks at s + correction (NULL: s); the outputs form `groups` equal groups of neighbours, a group counts as
 * its largest choice score and only the `keep` best groups can be chosen from; the `top` best are taken (ties to the lower index); weights = chosen s /
 * (their sum + 1e-20) * scale (normalise 0: s * scale).  A choice >= real is written as idx = real with weight 0, and idw[n] = the sum of such weights. */
int exl3_mix_topk_grouped(int32_t* idx, float* wts, float* idw, const float* logits, const float* correction, int kind, float scale, int normalise,
                          int groups, int keep, int n, int total, int real, int top, void* stream);

/* Ungated experts: hid[n*top + r] = act(Wu[e] h[n]) (EXL3_MIX_ACT_*).  In all experts' kernels a choice outside 0 .. experts-1 is skipped. */
int exl3_mix_moe_up_act(void* hid, const void* h, const void* wu, const int32_t* idx, int n, int top, int experts, int ff, int width, int act, int dtype, void* stream);
int exl3_mix_moe_expert_major_plain(void* per, void* hid, const void* h, const void* wu, const void* wd, const int32_t* idx,
                                    int n, int top, int experts, int ff, int width, int act, int dtype, void* stream);
/* exl3_mix_moe_down / exl3_mix_moe_combine with y[n] += idw[n] * h_id[n] (idw NULL: nothing added); combine skips the choices that idx (NULL: none)
 * places outside 0 .. experts-1. */
int exl3_mix_moe_down_id(void* y, const void* hid, const void* wd, const int32_t* idx, const float* wts, const void* h_id, const float* idw,
                         int n, int top, int experts, int ff, int width, int dtype, void* stream);
int exl3_mix_moe_combine_id(void* y, const void* sorted, const int32_t* where, const float* wts, const int32_t* idx, int experts, const void* h_id,
                            const float* idw, int n, int top, int width, int dtype, void* stream);

/* ---- parallel blocks over a layer norm, attention without softmax over paged keys, and recurrent mixers with a scalar decay per head ---- */

/* x[n] = table[tokens[n]] * scale + P(tok_pos[n]); P: entry 2i = sin(p freq[i]), entry 2i + 1 = cos(p freq[i]) (float32 angles). */
int exl3_mix_embed_sinusoid(float* x, const void* table, const int32_t* tokens, const int32_t* tok_pos, const float* freq, float scale, int n, int width, int vocab,
                            int dtype, void* stream);

/* h[i] = layer norm of residual row rows[i] (or i): (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b (b optional). */
int exl3_mix_layer_norm_rows(void* h, const float* x, const int32_t* rows, const float* w, const float* b, float eps, int n, int width, int dtype, void* stream);

/* The general form of exl3_mix_residual_rms.  mode 0: x stays; 1: x += y'; 2: x = y', with y' = (y + y2) * y_scale (y2 optional).  Then the norm of x:
 * center 0: x / sqrt(mean(x^2) + eps) * w; center 1: the layer norm with weight w and optional bias.  hn_out (optional) receives the normed rows; h
 * (optional) receives them too, or -- with conv_w [taps][width] and steps of one row per sequence -- normed row + its short causal convolution against
 * the slot's ring of the last taps - 1 normed rows, which is updated. */
int exl3_mix_residual_norm_conv(float* x, const void* y, int64_t y_ld, const void* y2, int64_t y2_ld, float y_scale, int mode, int center, const float* w,
                                const float* bias, float eps, void* h, int64_t h_ld, void* hn_out, int64_t hn_ld, const float* conv_w, int taps, void* ring,
                                const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, int n, int width, int dtype, void* stream);

/* exl3_mix_glu_act whose rows are also multiplied by sigmoid(rg[n]) (rg: one element per row, row stride rg_ld; may be null). */
int exl3_mix_glu_act_rowgate(void* out, const void* g, int64_t g_ld, const void* u, int64_t u_ld, const void* rg, int64_t rg_ld, int n, int ff, int kind, float limit,
                             int dtype, void* stream);

/* exl3_mix_topk_grouped with a group's score = the sum of its group_top largest choice scores (1: its largest). */
int exl3_mix_topk_grouped_ex(int32_t* idx, float* wts, float* idw, const float* logits, const float* correction, int kind, float scale, int normalise,
                             int groups, int keep, int group_top, int n, int total, int real, int top, void* stream);

/* Paged keys and values: pools k_pages [pages][page][kw], v_pages [pages][page][vw]; table [slots][table_ld] lists a sequence's pages in order.  Stores
 * the step's rows (row n at position tok_pos[n] of sequence tok_seq[n]). */
int exl3_mix_paged_store(void* k_pages, void* v_pages, const void* k, int64_t k_ld, const void* v, int64_t v_ld, const int32_t* table, int64_t table_ld, int page,
                         const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, int n, int kw, int vw, int dtype, void* stream);

/* Causal attention without softmax: out[n][h] = sum over the keys j <= n of the row's sequence of sigmoid(scale q.k_j + bias[h]) v_j.  Prompt steps read
 * the step's own keys (sequences start in the step); decode steps (one row per sequence) read the pages, len_after[n] keys. */
int exl3_mix_sigattn_prefill(void* out, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld, const float* bias,
                             const int32_t* cu, const int32_t* tok_seq, int n, int heads, int kv_heads, int dim, int vdim, float scale, int dtype, void* stream);
int exl3_mix_sigattn_decode(void* out, const void* q, int64_t q_ld, const void* k_pages, const void* v_pages, const float* bias, const int32_t* table, int64_t table_ld,
                            int page, const int32_t* slots, const int32_t* len_after, int n, int heads, int kv_heads, int dim, int vdim, float scale, int dtype, void* stream);
/* The same prompt step on the matrix cores (bfloat16; dim and vdim multiples of 16, dim <= 256, vdim <= 256). */
int exl3_mix_sigattn_prefill_mfma(void* out, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld, const float* bias,
                                  const int32_t* cu, int batch, int max_rows, int heads, int kv_heads, int dim, int vdim, float scale, void* stream);

/* mLSTM scan over the step's rows; state per slot: S [heads][vdim][dim], n [heads][dim], m [heads] (float32).  Sequences with pos0 == 0 start from zero
 * (m = 0).  zi / zf: the gate projections (one per head), bias_i / bias_f their biases; log gates are capped: cap tanh(. / cap).  o [n][heads][vdim] float32. */
int exl3_mix_mlstm_scan(float* o, float* S_state, float* n_state, float* m_state, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                        const void* zi, int64_t zi_ld, const void* zf, int64_t zf_ld, const float* bias_i, const float* bias_f,
                        const int32_t* cu, const int32_t* slots, const int32_t* pos0, int batch, int heads, int dim, int vdim, float q_scale, float cap,
                        int dtype, void* stream);

/* Gated delta rule: input stage (short convolutions with silu over x = q | k | v, unit query / key vectors, beta and decay; float32 results; ring
 * [slots][taps - 1][C] of the last rows of x) and the scan (state S [slots][heads][vdim][dim] float32; query / key head = head / (heads / kv_heads)). */
int exl3_mix_delta_prep(float* qo, float* ko, float* vo, float* beta, float* decay, const void* x, int64_t x_ld, const float* conv_w, int taps, void* ring,
                        const void* zb, int64_t zb_ld, const void* za, int64_t za_ld, const float* A_log, const float* dt_bias,
                        const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, const int32_t* pos0, const int32_t* len_after,
                        int n, int heads, int kv_heads, int dim, int vdim, float q_scale, int dtype, void* stream);
int exl3_mix_delta_scan(float* o, float* S_state, const float* q, const float* k, const float* v, const float* beta, const float* decay,
                        const int32_t* cu, const int32_t* slots, const int32_t* pos0, int batch, int heads, int kv_heads, int dim, int vdim, void* stream);

/* out[n][h] = o[n][h] / rms(o[n][h]) * w[(per_head ? h vdim : 0) ..] * gate(g[n][h]); gate 0: silu, 1: sigmoid. */
int exl3_mix_head_norm_gate(void* out, const float* o, const float* w, int per_head, const void* g, int64_t g_ld, int gate, float eps, int n, int heads, int vdim,
                            int dtype, void* stream);

/* out[n] = scale (a[n] / rms(a[n]) * wa + b[n] / rms(b[n]) * wb). */
int exl3_mix_rms_pair(void* out, const void* a, int64_t a_ld, const float* wa, const void* b, int64_t b_ld, const float* wb, float scale, float eps, int n, int width,
                      int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif
