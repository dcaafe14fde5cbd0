/*
 * litgpt_seq.h — C ABI of liblitgpt_seq.so: the MI355X (gfx950) kernels of the layered models (retention, latent-,
 * differential- and sink-attention, state-space and delta-rule mixers, gated and sparse feed-forwards, per-layer token
 * inputs) over an fp32 residual stream.
 *
 * Conventions: plain device pointers and sizes; every buffer is caller-owned; launches are asynchronous on `stream`
 * (graph-capturable); 0 on success, otherwise a hipError_t value with a message from lgs_last_error_string()
 * (thread-local). Activations are fp32. A weight matrix is [out][in], bf16 (w_f32 = 0: the activation operand is
 * rounded to bf16, sums are fp32) or fp32 (w_f32 = 1: plain fp32). Offsets and strides count elements.
 * A step is a packed batch: per token an int32 cache slot and position; per sequence its first row (seq_start,
 * B + 1 entries), slot and first position.
 */
#ifndef LITGPT_SEQ_H
#define LITGPT_SEQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* lgs_stream_t; /* == hipStream_t */

/* activations (lgs_linear epilogue, lgs_glu, lgs_head_gate, lgs_moe_up) */
#define LGS_ACT_NONE 0
#define LGS_ACT_RELU2 1     /* max(z, 0)^2 */
#define LGS_ACT_GELU_TANH 2 /* 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))) */
#define LGS_ACT_SILU 3
#define LGS_ACT_SIGMOID 4

const char* lgs_last_error_string(void);
int lgs_version(void);

/* y[z] (+)= act(a[z] w[z]^T) for z < batch: a[z] = a + z stride_a (M rows of K, row stride lda), w[z] = w + z stride_w
 * ([N][K]), y[z] = y + z stride_y (row stride ldy). M <= 8: streaming GEMV; otherwise 128x128 MFMA tiles (bf16) or
 * 64x64 FMA tiles (fp32). z_start (batch + 1 bounds, device) makes it grouped: batch z owns rows
 * [z_start[z], z_start[z+1]) of a list of at most M rows; list row i reads A row a_rows[i] (or i) and writes Y row i
 * (stride_a and stride_y are then ignored for the rows' place). a_bf16: A is a producer's bf16 copy (MFMA tiles with
 * bf16 weights only): the same values the fp32 stream would be rounded to, at half the operand traffic. y_bf16: the
 * result is written as bf16 (it feeds another bf16 product; MFMA tiles, no accumulate). */
int lgs_linear(const void* a, long lda, long stride_a, const void* w, int w_f32, long stride_w, void* y, long ldy,
               long stride_y, int M, int N, int K, int batch, int accumulate, int act, const int* a_rows,
               const int* z_start, int a_bf16, int y_bf16, lgs_stream_t stream);
/* x[t] = table[tokens[t]] * scale */
int lgs_embed(const int* tokens, const void* table, int w_f32, float scale, float* x, int T, int W, int vocab,
              lgs_stream_t stream);
/* x[t] = table[tokens[t]] * scale + pos_table[pos[t]] (both tables of one dtype); x_bf16: optional rounded copy */
int lgs_embed_pos(const int* tokens, const int* pos, const void* table, const void* pos_table, int w_f32, float scale,
                  float* x, void* x_bf16, int T, int W, int vocab, int positions, lgs_stream_t stream);
/* layer norm of a sublayer's output y [rows][n] joining the residual x [rows][n]:
 * x (+)= mult * ((y - mean) / sqrt(var + eps) * weight + bias), var = mean of the squared deviations (bias may be
 * NULL; accumulate 0 writes instead of adding); x_bf16: optional copy of the new x rounded to bf16 */
int lgs_layernorm(const float* y, const float* weight, const float* bias, float eps, float mult, int accumulate,
                  float* x, void* x_bf16, int rows, int n, lgs_stream_t stream);
/* z[i] = cap * tanh(z[i] / cap) in place */
int lgs_softcap(float* z, long n, float cap, lgs_stream_t stream);
/* group g of row r: y = x / sqrt(mean(x^2) + eps) * (offset + weight) (weight NULL: unit RMS), n values per group */
int lgs_rmsnorm(const float* x, long ldx, const float* weight, float offset, float eps, float* y, long ldy, int rows,
                int groups, int n, void* y_bf16 /* optional rounded copy, same layout */, lgs_stream_t stream);
int lgs_gather_rows(const float* x, const int* rows, float* y, int n_rows, int W, lgs_stream_t stream);

/* retention: rotary (pairs i, i + rot_dims/2; angle = position * inv_freq[i]) on q and k, k * k_scale, then per
 * sequence and head S <- decay S + k v^T, o = S^T q. state [slots][H][d][dv] fp32 is read unless the sequence's
 * first position is 0 and written back at the end of the step. d <= 512. chunked != 0 (and d <= 128) runs the
 * prompt form: chunks of 64 tokens as fp32 matrix products, the state carried from chunk to chunk in LDS; with a
 * workspace ws of B * max_chunks * H * d * dv floats (max_chunks = 64-token chunks of the longest sequence) the chunks
 * run side by side when sequences and heads alone would not fill the chip: local sums, a short carry over the
 * chunks, then the outputs. The prompt form rotates and scales q and k IN PLACE first (T_rows rows with positions
 * pos[T_rows]); the token-by-token form leaves them as they are. act (LGS_ACT_*): an activation on q, k and v as
 * projected, ahead of the rotation and the scale (the prompt form applies it in place, to v as well). */
int lgs_retention(float* q, float* k, float* v, long ld, float* state, const float* decay,
                  const float* inv_freq, const int* seq_start, const int* seq_slot, const int* seq_pos0, float* out,
                  int B, int H, int d, int dv, int rot_dims, float k_scale, int chunked, float* ws, int max_chunks,
                  int T_rows, const int* pos, int act, lgs_stream_t stream);
/* in place on o [T][H][dv]: (unit_norm ? o / rms(o) per head : o) * weight[i] * act(g[t * ldg + h * dv + i]) * post
 * (weight: dv values shared by the heads, or NULL). With w_g2 ([H dv][rank], bf16 or fp32 with g2_f32) g holds the
 * `rank` inner values of a low-rank gate per row and the gate's input is w_g2[h dv + i] . g[t * ldg ..]. */
int lgs_head_gate(float* o, const float* g, long ldg, int T, int H, int dv, int unit_norm, float eps, int act,
                  const float* weight, float post, void* o_bf16 /* optional rounded copy [T][H * dv] */,
                  const void* w_g2, int rank, int g2_f32, lgs_stream_t stream);
/* latent attention, per token: c = rmsnorm(proj[kv_off .. + r]) * norm_w -> cache_c[slot][pos] (bf16, or fp32 with
 * cache_f32); rotary (pairs 2i, 2i + 1) of proj[kv_off + r .. + dr] -> cache_kr[slot][pos] (fp32); the rotated
 * part of every head's query (at q_off + h (d + dr) + d) is rotated in place. */
int lgs_latent_prepare(float* proj, long ld, int q_off, int kv_off, void* cache_c, int cache_f32, float* cache_kr,
                       const float* norm_w, const float* inv_freq, const int* slot, const int* pos, int T, int H,
                       int d, int dr, int r, int rot_dims, int max_seq, float eps, lgs_stream_t stream);
/* out[t][h] = sum_j p_j c_j over cached rows j <= pos[t] of slot[t], p = softmax over
 * (qc[t][h] . c_j + q_rot[t][h] . kr_j) * scale with exp(sink[h]) added to the denominator (sink NULL: none).
 * r <= 1024, dr <= 128. splits > 1 spreads every (token, head)'s keys over that many workgroups (decode: few rows,
 * long contexts) and merges them in a second launch; part: T * H * splits * (r + 2) floats of workspace. */
int lgs_latent_attention(const float* qc, const float* proj, long ld, int q_off, const void* cache_c, int cache_f32,
                         const float* cache_kr, const float* sink, const int* slot, const int* pos, float* out, int T,
                         int H, int d, int dr, int r, int max_seq, float scale, int splits, float* part,
                         lgs_stream_t stream);
/* the prompt form of lgs_latent_attention: tiles of 16 consecutive tokens of one sequence and one head against key
 * tiles of 16 cached rows, both products on fp32 MFMA; max_len = the most tokens any sequence brings. r % 64 == 0. */
int lgs_latent_attention_tiles(const float* qc, const float* proj, long ld, int q_off, const void* cache_c,
                               int cache_f32, const float* cache_kr, const float* sink, const int* seq_start,
                               const int* seq_slot, const int* seq_pos0, float* out, int B, int max_len, int H, int d,
                               int dr, int r, int max_seq, float scale, lgs_stream_t stream);

/* out[t][i] = act(a[t * ld + i]) * b[t * ld + i], i < n */
int lgs_glu(const float* a, const float* b, long ld, void* out /* fp32, or bf16 with out_bf16 */, int out_bf16, int T,
            int n, int act, lgs_stream_t stream);
/* per token: ids / wts [T][top] = the top largest of z[t * ld .. + E] (lowest index first among equals) and the
 * softmax over those. E <= 256. */
int lgs_moe_route(const float* z, long ld, int T, int E, int top, int* ids, float* wts, lgs_stream_t stream);
/* per token: s = softmax(z[t * ld .. + E]) over all E outputs; ids = the top largest of s + bias (bias NULL: of s;
 * lowest index first among equals), wts = s at those places (not renormalised). E <= 256. */
/* sigmoid != 0: s = sigmoid(z) of every output on its own instead of the softmax. square != 0: wts = s^2 (the weight
 * of an expert whose INPUT is scaled by s when its activation is the square of relu). */
int lgs_moe_route_scores(const float* z, long ld, int T, int E, int top, const float* bias, int* ids, float* wts,
                         int sigmoid, int square, lgs_stream_t stream);
/* out[t][i] = act(a[t * ld + i]) * (gate ? sigmoid(gate[t * ldg]) : 1), i < n: the activation of an ungated unit whose
 * up-projection is part of a fused product, with an optional gate of one number per row */
int lgs_act_rows(const float* a, long ld, const float* gate, long ldg, void* out /* fp32, or bf16 with out_bf16 */,
                 int out_bf16, int T, int n, int act, lgs_stream_t stream);
/* the router product z = w h[t] (w [E][K], fp32 sums) and lgs_moe_route_scores' routing in one launch: the form of
 * steps with few tokens */
int lgs_moe_router(const float* h, long ldh, const void* w, int w_f32, int T, int K, int E, int top, const float* bias,
                   int* ids, float* wts, int sigmoid, int square, lgs_stream_t stream);
/* streaming experts: actbuf[t * top + k] = act(up[ids[t][k]] h[t]), or with gated (up holds per expert F gate rows,
 * then F up rows) act(gate h) * (up h); x[t] (+)= sum_k wts[t][k] down[ids[t][k]] actbuf[..]. An id >= n_real names
 * an identity expert without matrices: it is skipped by lgs_moe_up and contributes wts * hin[t] in lgs_moe_down. */
int lgs_moe_up(const float* h, long ldh, const void* up, int w_f32, const int* ids, float* actbuf, int T, int top,
               int F, int K, int act, int gated, int n_real, lgs_stream_t stream);
int lgs_moe_down(const float* actbuf, const void* down, int w_f32, const int* ids, const float* wts, float* x,
                 long ldx, int T, int top, int N, int F, int n_real, const float* hin, long ldh, int accumulate,
                 lgs_stream_t stream);
/* counting sort of the (token, choice) pairs by expert: z_start [E + 1], tok_of [pairs] (token of each sorted entry),
 * where [pairs] (sorted place of each pair); the order inside an expert's range is not fixed. ws: 2 E ints, zero on
 * entry, left zero. */
int lgs_moe_sort(const int* ids, int pairs, int top, int E, int* z_start, int* tok_of, int* where, int* ws,
                 lgs_stream_t stream);
/* x[t] (+)= sum_k wts[t][k] * y[where[t * top + k]]; with ids, a choice with ids[t][k] >= n_real (an identity expert)
 * contributes hin[t] instead of a row of y */
int lgs_moe_combine(const float* y, const int* where, const float* wts, float* x, long ldx, int T, int top, int N,
                    const int* ids, int n_real, const float* hin, long ldh, int accumulate, lgs_stream_t stream);
/* x[t] += unit_rms(proj_w (gelu_tanh(gate_w x[t]) * table[tokens[t]][col0 .. + dim])) * norm_w */
int lgs_token_side(float* x, const int* tokens, const void* table, int w_f32, long ld_table, int col0,
                   const void* gate_w, const void* proj_w, const float* norm_w, int T, int W, int dim, int vocab,
                   float eps, lgs_stream_t stream);

/* ---- several residual streams (hyper-connections) ---- */
/* x[t][j] = table[tokens[t]] * scale for each of `streams` streams: x is [T][streams][W] */
int lgs_embed_streams(const int* tokens, const void* table, int w_f32, float scale, float* x, int T, int W, int vocab,
                      int streams, lgs_stream_t stream);
/* One sublayer boundary on x [T][streams][W], in place. With y [T][W] (a sublayer's output):
 * x_j <- sum_i mix[i * streams + j] x_i + out[j] y. Then, with `in`: u = sum_j in[j] x_j,
 * h = u / sqrt(mean(u^2) + eps) * norm_w (h_bf16: optional rounded copy), or h = u itself when norm_w is NULL.
 * Either half may be left out (y or in NULL). streams <= 8; mix / out / in are fp32 on the device. */
int lgs_streams_step(float* x, const float* y, const float* mix, const float* out, const float* in,
                     const float* norm_w, float* h, void* h_bf16, float eps, int T, int W, int streams,
                     lgs_stream_t stream);

/* ---- differential attention ---- */
/* Per token: rotary (interleaved pairs 2i, 2i + 1 of the first rot_dims dims of every map; angle = position *
 * inv_freq[i]) on the 2 H query maps at proj[q_off ..] in place and on the 2 G key maps at proj[k_off ..] on their way
 * to cache_k [slots][max_seq][G][2 d]; the values at proj[v_off ..] go to cache_v [slots][max_seq][G][dv]. The caches
 * are bf16, or fp32 with cache_f32. k_off < 0: queries only (the layer attends over another layer's cache). */
int lgs_diffattn_prepare(float* proj, long ld, int q_off, int k_off, int v_off, void* cache_k, void* cache_v,
                         int cache_f32, const float* inv_freq, const int* slot, const int* pos, int T, int H, int G,
                         int d, int dv, int rot_dims, int max_seq, lgs_stream_t stream);
/* out[t][h] = post * unit_rms(a1 - lambda a2), a_m = softmax_j(cap(q_m . k_m,j * scale)) V over the cached rows
 * lo <= j <= position of the sequence's slot, lo = position - position % chunk (chunk 0: lo = 0);
 * cap(s) = cap tanh(s / cap) (cap 0: none); query head h reads key head h / (H / G). q: the rotated queries
 * (row stride ld, 2 d per head). max_len: the most tokens a sequence brings; with max_len 1 the keys of a
 * (token, head) may be spread over `splits` workgroups (part: T H splits (4 + 2 dv) floats). dv <= 256. */
int lgs_diffattn(const float* q, long ld, const void* cache_k, const void* cache_v, int cache_f32, const int* seq_start,
                 const int* seq_slot, const int* seq_pos0, float* out, void* out_bf16, float* part, int splits, int B,
                 int max_len, int H, int G, int d, int dv, int max_seq, int chunk, float scale, float cap, float lambda,
                 float eps, float post, lgs_stream_t stream);

/* ---- softmax attention with one map per head: normed and / or rotated queries and keys, a sink, a head gate ---- */
/* Per token: every query head at proj[q_off ..] is (norm != 0) divided by its root mean square (eps inside the root)
 * and multiplied by q_w [d] (NULL: no weight), then rotated on the pairs (i, i + rot_dims / 2) by position *
 * inv_freq[i] (rot_dims 0: not), then multiplied by the query temperature
 * 1 + temp_coef * ln(floor((position + 1) / temp_every) + 1) (temp_every 0: 1), in place; every key head at
 * proj[k_off ..] is normed (k_w) and rotated alike on its way to cache_k [slots][max_seq][G][d], the projection
 * itself stays as it is; the values at proj[v_off ..] go to cache_v [slots][max_seq][G][dv] (bf16, or fp32);
 * v_off == k_off with dv == d makes the values the keys as projected. */
int lgs_normattn_prepare(float* proj, long ld, int q_off, int k_off, int v_off, void* cache_k, void* cache_v,
                         int cache_f32, const int* slot, const int* pos, int T, int H, int G, int d, int dv, int max_seq,
                         float eps, float temp_coef, int temp_every, int norm, const float* q_w, const float* k_w,
                         const float* inv_freq, int rot_dims, lgs_stream_t stream);
/* out[t][h] = post * sum_j p_j v_j over the cached rows j of the mask (as lgs_diffattn's), p = softmax of
 * cap((q . k_j) * scale) with exp(sink[h]) added to the normaliser (sink NULL: none); grouped key / value heads.
 * One map per head: q rows hold d values per head. max_len, splits and part (T H splits (2 + dv) floats) as in
 * lgs_diffattn. gate (NULL: none): head h's output at row t is multiplied by sigmoid(gate[t * ldg + h]). */
int lgs_sinkattn(const float* q, long ld, const void* cache_k, const void* cache_v, int cache_f32, const float* sink,
                 const int* seq_start, const int* seq_slot, const int* seq_pos0, float* out, void* out_bf16, float* part,
                 int splits, int B, int max_len, int H, int G, int d, int dv, int max_seq, int chunk, float scale,
                 float cap, float post, const float* gate, long ldg, lgs_stream_t stream);

/* ---- gated delta rule ---- */
/* Per token, on rows qkv [T][ld] = q [G][d] | k [G][d] | v [H][dv] (after their convolution): q and k become unit
 * vectors per head, x / sqrt(sum(x^2) + norm_eps), q also times q_scale, in place; beta[t][h] = sigmoid(b[t ldb + h]);
 * dec = exp(-exp(A_log[h]) softplus(a + dt_bias)) with a, dt_bias and dec per head and key channel ([H][d],
 * per_channel) or per head ([H]); kq[t][g] = k . q of the prepared vectors of key head g.
 * unit 0: k stays as projected and q is only multiplied by q_scale. decay_form 1: dec = sigmoid(a + dt_bias)^(1 / tau)
 * (A_log unused). b NULL: no betas (the plain rule of lgs_gated_delta). */
int lgs_delta_prepare(float* qkv, long ld, const float* a, long lda, const float* b, long ldb, const float* A_log,
                      const float* dt_bias, float* dec, float* beta, float* kq, int T, int H, int G, int d,
                      int per_channel, float q_scale, float norm_eps,
                      const void* w_a2 /* optional: a holds `rank` values per row, the raw input of entry i is w_a2[i] . a */,
                      int rank, int a2_f32, int unit, int decay_form, float tau, lgs_stream_t stream);
/* The same for a step in which every sequence brings ONE token (row b of u belongs to sequence b), with the short
 * causal convolution + silu of the C = 2 G d + H dv channels of u in the same launch: conv_w [C][taps] (column
 * taps - 1 weights the token itself, no bias), conv_state [slots][taps - 1][C] as in lgs_conv_silu (read unless the
 * sequence starts at position 0, shifted by one token). qkv [B][C] receives the prepared row. */
int lgs_delta_step_prepare(const float* u, long ldu, const void* conv_w, int conv_f32, int taps, float* conv_state,
                           const int* seq_slot, const int* seq_pos0, float* qkv, const float* a, long lda, const float* b,
                           long ldb, const float* A_log, const float* dt_bias, float* dec, float* beta, float* kq, int B,
                           int H, int G, int d, int dv, int per_channel, float q_scale, float norm_eps, const void* w_a2,
                           int rank, int a2_f32, lgs_stream_t stream);
/* Per sequence and head, token by token: S <- diag(dec) S; u = beta (v - S^T k); S <- S + k u^T; out = S^T q
 * (evaluated as S'^T q + u kq on the decayed state S', kq [T][G] = k . q from lgs_delta_prepare).
 * Head h reads q / k head h / (H / G). state [slots][H][d][dv] fp32 is read unless the sequence starts at position 0
 * and written back. d <= 512. lanes: lanes that share a state column (4, 8 or 16; 0: chosen from the sizes).
 * plain != 0: the gated rule without the correction, S <- diag(dec) S + k v^T, out = S^T q (beta unused). */
int lgs_gated_delta(const float* qkv, long ld, const float* dec, const float* beta, const float* kq, float* state,
                    const int* seq_start, const int* seq_slot, const int* seq_pos0, float* out, int B, int H, int G, int d,
                    int dv, int per_channel, int lanes, int plain, lgs_stream_t stream);

/* ---- selective state-space mixer ---- */
/* out[t][c] = silu(bias[c] + sum_j w[c][j] u[t - (taps - 1 - j)][c]) per sequence of a packed batch; inputs before
 * the step come from state [slots][taps - 1][C] (oldest first; zeros when the sequence starts at position 0), which
 * is left holding the step's last taps - 1 inputs. taps <= 16. */
int lgs_conv_silu(const float* u, long ld, const void* w, const void* bias, int w_f32, float* state,
                  const int* seq_start, const int* seq_slot, const int* seq_pos0, float* out, int B, int max_len, int C,
                  int taps, lgs_stream_t stream);
/* Per sequence and head: dt = softplus(dt_raw + dt_bias), S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x.
 * xbc rows hold x [heads][dv] | B [groups][N] | C [groups][N]; head h reads group h / (heads / groups).
 * state [slots][heads][N][dv] fp32 is read unless the sequence starts at position 0, and written back. N <= 256.
 * With a workspace (ws: B max_chunks heads N dv floats, wdec: B max_chunks heads floats; max_chunks = 64-token chunks
 * of the longest sequence; N <= 128) the prompt form runs: chunks as fp32 matrix products side by side, a short
 * carry over the chunks, then the outputs. Without (ws NULL) the tokens are walked one by one. */
int lgs_ssm_scan(const float* xbc, long ldx, const float* dt, long ldd, const float* dt_bias, const float* A_log,
                 const float* D, float* state, const int* seq_start, const int* seq_slot, const int* seq_pos0,
                 float* y, int B, int heads, int groups, int N, int dv, float* ws, float* wdec, int max_chunks,
                 lgs_stream_t stream);
/* out = v / sqrt(mean over the group of v^2 + eps) * w, v = y * silu(z); `groups` equal parts of `inner` columns */
int lgs_gated_group_norm(const float* y, const float* z, long ldz, const float* w, float eps, float* out,
                         void* out_bf16, int T, int inner, int groups, lgs_stream_t stream);
/* out[t][i] = g sigmoid(alpha g) (u + shift), g = min(a[t ld + i], limit), u = clamp(b[t ld + i], -limit, limit)
 * (limit <= 0: no clamps) */
int lgs_glu_clamped(const float* a, const float* b, long ld, void* out, int out_bf16, int T, int n, float alpha,
                    float limit, float shift, lgs_stream_t stream);

/* ---- sandwich norms ---- */
/* One boundary between two sublayers whose input AND output are normed, rows of n values. With y0 (the sublayer that
 * ran; y1: an optional second branch): b_i = w_i ? y_i / rms(y_i) * w_i : y_i, s = coef * (b_0 + b_1),
 * x += s / rms(s) * post_w (post_w: the output norm's weight times the layer's per-channel scale). Then with next_w:
 * h = x / rms(x) * next_w, the next sublayer's input, as fp32 (h) and / or rounded to bf16 (h_bf16). */
int lgs_sandwich_step(float* x, const float* y0, const float* w0, const float* y1, const float* w1, float coef,
                      const float* post_w, const float* next_w, float* h, void* h_bf16, float eps, int rows, int n,
                      lgs_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif
