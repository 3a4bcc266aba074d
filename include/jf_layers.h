/* jf_layers.h — C ABI of libjf_layers.so: layer kernels for decoders with a 32-bit residual stream, served over a paged
 * key/value pool and per-request state slots.  Device pointers + sizes, stream as void*.  Activation tensors are row-major
 * float or bfloat16 (`dtype`: JL_F32 / JL_BF16) with an explicit row stride in elements where a tensor is a column range of a
 * wider matrix; residual stream, router, probabilities and recurrent state are float.  Every function returns JL_OK or a
 * negative code (jl_last_error() has the text) and only enqueues work on `stream`.
 *
 * A step's tokens are one ragged batch: N token rows, the rows of one request consecutive and in position order.  Per request
 * b the int32 record seq[b] = {row0, count, pos0, slot}: its first row, its number of rows, the position of its first row
 * (= tokens already cached) and its state slot. */
#ifndef JF_LAYERS_H
#define JF_LAYERS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define JL_API __attribute__((visibility("default")))
#define JL_VERSION 124
#define JL_OK 0
#define JL_E_INVALID (-1)
#define JL_E_LAUNCH (-3)
#define JL_F32 0
#define JL_BF16 1

JL_API int jl_version(void);
JL_API const char *jl_last_error(void);

/* x[n, :] = embed[ids[n], :] * scale (float); x0, when given, receives the same rows (the embedding output a repeated pass adds
 * again). */
JL_API int jl_embed_scale(const void *embed, int dtype, const int64_t *ids, int64_t N, int32_t W, float scale, float *x, float *x0,
                          void *stream);

/* Residual update + RMS norm: x[n] += sum_{s < y_count} y[n * y_count + s] (y of dtype y_dtype, may be null) + x0[n] (float,
 * may be null); then, when `out` is given, out[n] = x[n] / sqrt(mean(x[n]^2) + eps) * w (w of `dtype`, null = no weight). */
JL_API int jl_add_rmsnorm(float *x, const void *y, int y_dtype, int32_t y_count, const float *x0, const void *w, float eps,
                          void *out, int dtype, int64_t N, int32_t W, void *stream);

/* Residual update from several scaled addends, then up to two RMS norms of the SAME updated row with float weights stored around
 * `w_offset` — the layer whose mixer and feed-forward both read one stream and are added in one sum:
 *   x[n, c] += sum_a scale_a[c] * sum_{s < count_a} y_a[(n * count_a + s), c]        (at most 3 addends; scale null = 1)
 *   out1[n] = x[n] / sqrt(mean(x[n]^2) + eps) * (w_offset + w1);   out2 likewise with w2   (out1 / out2 / w1 / w2 may be null)
 * x float in place; y_a of its own dtype; out1 / out2 of `dtype`; out2_f32 (may be null) receives the second norm unrounded as well
 * (what a float router reads beside the bfloat16 copy the experts' products read). */
typedef struct { const void *y; int32_t dtype; int32_t count; const float *scale; } jl_addend;
JL_API int jl_scaled_add_norms(float *x, const jl_addend *addends, int32_t n_addends, const float *w1, const float *w2, float w_offset,
                               float eps, void *out1, void *out2, float *out2_f32, int dtype, int64_t N, int32_t W, void *stream);

/* Gated activation of a feed-forward whose gate and linear branch are column ranges of one product z [N, ld] (F columns each at
 * g_col / u_col):   out[n, c] = act(g) * lin(u) * sigmoid(row_gate[n * rg_ld])        (row_gate null: no row gate)
 *   JL_ACT_GELU_TANH:      act(g) = 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))), lin(u) = u
 *   JL_ACT_CLAMPED_SWISH:  g' = min(g, limit), u' = clamp(u, -limit, limit); act = g' sigmoid(alpha g'), lin = u' + shift
 * u_col < 0: the unit has no linear branch (out = act(g), a plain activation).
 * z, row_gate and out [N, F] of `dtype`; the arithmetic is float. */
#define JL_ACT_GELU_TANH 0
#define JL_ACT_CLAMPED_SWISH 1
#define JL_ACT_SILU 2             /* act(g) = g sigmoid(g), lin(u) = u */
#define JL_ACT_GELU_ERF 3         /* act(g) = 0.5 g (1 + erf(g / sqrt 2)), lin(u) = u */
#define JL_ACT_NONE (-1)          /* where an activation is optional (jl_short_conv) */
JL_API int jl_gated_act(const void *z, int dtype, int64_t N, int64_t ld, int32_t g_col, int32_t u_col, int32_t F, int32_t kind, float limit,
                        float alpha, float shift, const void *row_gate, int64_t rg_ld, void *out, void *stream);

/* Whole-projection query / key norm + cache append.  proj [N, ld] holds q (H*D columns at q_col), k (G*D at k_col) and v (G*Dv at
 * v_col).  q_out [N, H*D] = rms_norm(q) * wq over ALL H*D columns at once; the key is normalised the same way over G*D with wk and
 * stored at k_cache[slot[n]] ([pool tokens, G*D]); v is stored as it is at v_cache[slot[n]] ([pool tokens, G*Dv]).  slot < 0 skips
 * the stores. */
JL_API int jl_qk_norm_append(const void *proj, int dtype, int64_t N, int64_t ld, int32_t q_col, int32_t k_col, int32_t v_col,
                             int32_t H, int32_t G, int32_t D, int32_t Dv, const void *wq, const void *wk, float eps, void *q_out,
                             void *k_cache, void *v_cache, const int64_t *slot, void *stream);

/* Attention over the paged pool with a sliding window that keeps the first tokens, a bucketed distance bias and mixed heads:
 *   visible(i, j) = j <= i and (i - j < window or j < keep_first)
 *   s_g(i, j) = q_g(i) . k_c(g)(j) * scale + rel[lut[min(i - j, lut_len - 1)], g]          (c(g) = g / (H / G))
 *   p_g(i, .) = softmax over the visible j;   w_h(i, j) = sum_g talk[h, g] p_g(i, j)  (talk null: w = p)
 *   out_h(i) = (sum_j w_h(i, j) v_c(h)(j)) * sigmoid(gate_h(i))                             (gate null: no gate)
 * With `sink` (float [H], may be null) the softmax's denominator of head g holds one more term exp(sink[g]): an extra
 * score that attends to nothing (taken as it is: no scale, no bias; present exactly once per row), so a row's weights sum to less than one.  `gate` is read element by element
 * ([N, H*Dv], rows gate_ld apart) or, with gate_heads != 0, one number per head ([N, H], rows gate_ld apart).
 * tiles [n_tiles, 4] int32 = {b, first query position, count (<= TQ), first row}: consecutive rows of one request;
 * block_tables [*, bt_stride] int32 pages of request b in order; a key j lives at token page * page_size + j % page_size of the
 * pool.  window <= 0 means no window (plain causal).  rel [rows, H] float and lut int32 may be null (no bias). */
typedef struct {
    const void *q; const void *gate; int64_t gate_ld; const void *k_cache; const void *v_cache; void *out;
    const int32_t *block_tables; const int32_t *tiles; const float *rel; const int32_t *lut; const float *talk;
    int32_t bt_stride, n_tiles, lut_len, page_size, H, G, D, Dv, window, keep_first, TQ, dtype;
    float scale;
    int32_t splits, n_rows;       /* splits > 1 (TQ 32 only): each tile's keys are shared out over `splits` workgroups — statistics, */
    float *scratch;               /* outputs, join: three launches; scratch of jl_attn_scratch_floats() floats, n_rows = N          */
    void *q_pack;                 /* TQ 32 only: room for n_tiles * 32 * H * D elements (the queries in matrix-operand order)        */
    /* Pools that are column ranges of wider rows, fewer value heads than key heads, float outputs (all 0 = as described above): */
    int64_t k_ld, v_ld;           /* row stride of k_cache / v_cache in elements (0: G*D / Gv*Dv).  v_cache may point into k_cache.    */
    int32_t Gv;                   /* value heads (0: G).  G % Gv == 0; key head c reads value head c % Gv (score maps share values)   */
    int32_t out_dtype;            /* dtype of `out` when it differs from `dtype`: JL_OUT_F32 = float outputs from bfloat16 inputs     */
    const float *sink;            /* float [H] or null: one more term exp(sink[g]) in head g's softmax denominator                    */
    int32_t gate_heads;           /* != 0: `gate` holds one number per head ([N, H]) instead of one per output element                */
} jl_attn_args;
#define JL_OUT_SAME 0
#define JL_OUT_F32 2
JL_API int64_t jl_attn_scratch_floats(int32_t n_tiles, int32_t n_rows, int32_t H, int32_t Dv, int32_t splits);
JL_API int jl_attn_window(const jl_attn_args *a, void *stream);
/* TQ (query rows per tile) the kernel wants for this dtype, these sizes and these pool row strides (0: dense rows); 0 when
 * they do not fit */
JL_API int jl_attn_tile_rows(int dtype, int32_t H, int32_t G, int32_t D, int32_t Dv, int64_t k_ld, int64_t v_ld);

/* The same attention without bias and head mixing (sink and gate as above), in ONE sweep over the keys on the matrix cores, for heads in groups that
 * share a key head (H / G query heads per key head c, value head c % Gv): bfloat16, D % 8 == 0 up to 640, Dv % 32 == 0 up to 512,
 * row strides % 4 == 0.  v_cache == k_cache (with G = 1, Dv <= D): the values are the first Dv columns of the key rows — the pool
 * of latent attention — and are not loaded a second time.  Of jl_attn_args it reads q, k_cache, v_cache, k_ld, v_ld, out, out_dtype,
 * block_tables, bt_stride, tiles, n_tiles, page_size, H, G, Gv, D, Dv, window, scale, dtype, sink, gate, gate_ld, gate_heads, splits, scratch and TQ, which must be
 * what jl_attn_sweep_tile_rows returns (0: sizes not taken).  splits in 2 .. 64: the keys of every tile are shared out over that
 * many workgroups and joined by a second launch; `scratch` then holds jl_attn_sweep_scratch_floats floats. */
JL_API int jl_attn_sweep(const jl_attn_args *a, void *stream);
JL_API int jl_attn_sweep_tile_rows(int dtype, int32_t H, int32_t G, int32_t Gv, int32_t D, int32_t Dv, int64_t k_ld, int64_t v_ld,
                                   int32_t v_in_k);
JL_API int64_t jl_attn_sweep_scratch_floats(int32_t n_tiles, int32_t H, int32_t G, int32_t Dv, int32_t splits);
/* Long portions: with tiles of jl_attn_sweep_wide_tile_rows queries (0: sizes not taken — key widths up to 256, value widths up to 128) and
 * splits <= 1, jl_attn_sweep runs the form in which a workgroup owns up to 128 (query, head) rows and every wavefront keeps its 32
 * rows to itself (scores, weights and outputs never leave its registers). */
JL_API int jl_attn_sweep_wide_tile_rows(int dtype, int32_t H, int32_t G, int32_t Gv, int32_t D, int32_t Dv, int64_t k_ld, int64_t v_ld,
                                        int32_t v_in_k);

/* Residual update, weighted sum over the streams of all depths, RMS norm — the layer whose result is kept beside the results of all
 * layers before it, and whose successor reads a learned mixture of them:
 *   y[n] = x_in[n] + mult * sum_a scale_a * sum_s y_a[n, s]                       (addends as for jl_scaled_add_norms; at most 3)
 *   depth >= 0:  streams[depth][n] = y[n];  x_out[n] = sum_{j <= depth} mix[j] * streams[j][n]   (mix null: x_out = y)
 *   depth <  0:  x_out[n] = y[n]              (no addends: nothing is stored, the norm reads x_in)
 *   out[n] = x_out[n] / sqrt(mean(x_out[n]^2) + eps) * w     in `dtype`, and / or unrounded in out_f32 (either may be null; w null = 1)
 * streams: float, stream j at streams + j * stream_ld.  x_out may be x_in but must not lie inside streams[0 .. depth].
 * With shift_mu (float [W]) the launch also does jl_token_shift's work, for a step in which EVERY request brings one row (N = B, row n is
 * request n of seq [B, 4]): out_shift[n] = h + (tail[slot] - h) * shift_mu with h the unrounded norm (no tail before position 0), and
 * tail[slot] = h. */
JL_API int jl_depth_mix_norm(const float *x_in, const jl_addend *addends, int32_t n_addends, float mult, float *streams, int64_t stream_ld,
                             int32_t depth, const float *mix, float *x_out, const float *w, float eps, void *out, int dtype, float *out_f32,
                             int64_t N, int32_t W, const float *shift_mu, const int32_t *seq, float *shift_tail, void *out_shift, void *stream);

/* Token shift: out[t] = h[t] + (h[t-1] - h[t]) * mu, element by element, h float [N, W], mu float [W], out [N, W] of `dtype`.  h[t-1] of
 * a request's first row is tail[slot] (float [slots, W]) when the request has a past (pos0 > 0) and zero otherwise; tail[slot] then
 * becomes the h of the request's last row of this step.  row_req [N] int32, seq [B, 4] as above. */
JL_API int jl_token_shift(const float *h, const float *mu, const int32_t *row_req, const int32_t *seq, float *tail, int64_t N, int32_t W,
                          void *out, int dtype, void *stream);

/* z <- cap * tanh(z / cap) in place over `total` floats (soft cap of the logits). */
JL_API int jl_softcap(float *z, int64_t total, float cap, void *stream);

/* Sublayer-output norm + residual update: x[n] += y[n] / sqrt(mean(y[n]^2) + eps) * g[0] (x float in place, y of y_dtype, g one
 * float); when `out` is given, out[n] = x[n] in `out_dtype` (what the next sublayer's product reads). */
JL_API int jl_norm_add(float *x, const void *y, int y_dtype, const float *g, float eps, void *out, int out_dtype, int64_t N, int32_t W,
                       void *stream);

/* Polynomial activation with unit-RMS powers: out = c0 n(z) + c1 n(z^2) + c2 n(z^3) + c3, powers element by element,
 * n(u) = u / sqrt(mean(u^2) + eps) over the row's F values.  z, out [N, F] of `dtype`; coef four floats. */
JL_API int jl_polynorm(const void *z, int dtype, int64_t N, int32_t F, const float *coef, float eps, void *out, void *stream);

/* Causal depthwise convolution over time, added to its input, with the request's last inputs carried in its slot:
 *   out[t, c] = x[t, c] + sum_{j < taps} w[c, j] * x[t - taps + 1 + j, c]        (zeros before the sequence's start)
 * x float [N, W]; w [W, taps] and out [N, W] of `dtype`; row_req [N] int32 the request of every row; seq [B, 4] as above;
 * tail float [slots, taps - 1, W]: the inputs at positions pos0 - taps + 1 .. pos0 - 1 of the slot's request (entries before
 * position 0 are never read, so a slot's old content does not matter to a new request).  jl_causal_conv reads the tail and, for a
 * request with ONE row in the step, moves it on; jl_causal_conv_carry, enqueued after it, does that for the requests with more rows
 * (not needed when no request has more than one).  taps <= JL_CONV_MAX_TAPS. */
#define JL_CONV_MAX_TAPS 16
JL_API int jl_causal_conv(const float *x, const void *w, int dtype, const int32_t *row_req, const int32_t *seq, float *tail,
                          int64_t N, int32_t W, int32_t taps, void *out, void *stream);
JL_API int jl_causal_conv_carry(const float *x, const int32_t *seq, int32_t B, float *tail, int32_t W, int32_t taps, void *stream);

/* Short causal convolution over time of a column range of a product, with an activation and no residual:
 *   out[t, c] = act(sum_{j < taps} w[c, j] * x[t - taps + 1 + j, col + c])        (zeros before the sequence's start)
 * x [N, ld] and w [C, taps] of `dtype`, out float [N, C]; act JL_ACT_SILU or JL_ACT_NONE; taps <= 8.  tail float [slots, taps - 1, C] as for
 * jl_causal_conv (the INPUTS at the positions before the step); it is moved on here as well — for requests with one row in the launch
 * itself, for the others (max_count > 1) by a second launch enqueued behind it. */
JL_API int jl_short_conv(const void *x, int dtype, int64_t ld, int32_t col, const void *w, const int32_t *row_req, const int32_t *seq, int32_t B,
                         int32_t max_count, float *tail, int64_t N, int32_t C, int32_t taps, int32_t act, float *out, void *stream);

/* Per-head query / key stage for attention with M score maps per head: rotation, norm, query temperature, cache append.  proj
 * [N, ld] holds q (H heads x M maps x D at q_col, head by head), k (G x M x D at k_col) and v (G x Dv at v_col).  With rot_dims > 0
 * every D-vector is first rotated by its position p = pos[n]: of its first rot_dims dimensions, i and i + rot_dims/2 form a pair
 * (u, v) -> (u cos a - v sin a, v cos a + u sin a), a from the cos / sin tables [positions, rot_dims/2] float; the rest pass unchanged.
 * Every D-vector is then RMS-normalised on its own and multiplied by wq / wk [D] (null: no weight); the query is further multiplied by
 * 1 + t_coef * ln(floor((p + 1) / t_every) + 1) (t_coef 0: no temperature).  Queries and keys are written MAP-major — q_out [N, M, H, D], k_cache[slot[n]] = [M, G, D] — so that
 * query row m*H + h reads key row (m*H + h) / (H/G) = m*G + h/(H/G) and value head (m*G + g) % G: one attention launch with M*H query
 * heads, M*G key heads and G value heads computes all maps.  With maps_apart != 0 the queries are written [M, N, H, D] instead: one
 * launch per map, each over its own G*D columns of the key rows.  v goes to v_cache[slot[n]] as it is. */
JL_API int jl_head_norm_append(const void *proj, int dtype, int64_t N, int64_t ld, int32_t q_col, int32_t k_col, int32_t v_col, int32_t H,
                               int32_t G, int32_t M, int32_t D, int32_t Dv, const void *wq, const void *wk, float eps, float t_coef,
                               int32_t t_every, const int32_t *pos, void *q_out, int32_t maps_apart, void *k_cache, void *v_cache,
                               const int64_t *slot, int32_t rot_dims, const float *cos_t, const float *sin_t, void *stream);

/* Differential combination of two score maps' outputs a1, a2 (float, rows of H*Dv values `ld` floats apart):
 * o = a1 - lambda * a2;  out[n, h] = o / sqrt(mean(o^2) + eps) * out_scale over the head's Dv values; out [N, H*Dv] of `dtype`. */
JL_API int jl_diff_combine(const float *a1, const float *a2, int64_t ld, int64_t N, int32_t H, int32_t Dv, float lambda, float eps,
                           float out_scale, void *out, int dtype, void *stream);

/* Latent attention, input side.  proj [N, ld] holds the query latent (Rq columns at q_col) and the key/value latent (R columns at
 * kv_col) followed by rd rotary key dimensions shared by all heads.
 *   cq_out [N, Rq] = rms_norm(query latent) * wq
 *   pool[slot[n]] = [rms_norm(key/value latent) * wkv (R) | rotate(rotary key, pos[n]) (rd)]          (pool rows of R + rd)
 * rotate: of the first rot_dims dimensions, i and i + rot_dims/2 form a pair (u, v) -> (u cos a - v sin a, v cos a + u sin a),
 * a from the cos / sin tables [positions, rot_dims/2] float; the rest pass unchanged (`pairing` JL_ROT_NEIGHBOURS: 2i and 2i + 1 form
 * the pair instead).  Rq = 0: the model has no query latent (wq, cq_out null; nothing is read at q_col). */
#define JL_ROT_HALVES 0          /* dimension i pairs with i + rot_dims/2 */
#define JL_ROT_NEIGHBOURS 1      /* dimension 2i pairs with 2i + 1 (angle i) */
JL_API int jl_latent_prep(const void *proj, int dtype, int64_t N, int64_t ld, int32_t q_col, int32_t Rq, int32_t kv_col, int32_t R,
                          int32_t rd, int32_t rot_dims, const void *wq, const void *wkv, float eps, const int32_t *pos,
                          const float *cos_t, const float *sin_t, int64_t table_len, void *cq_out, void *pool, const int64_t *slot,
                          int32_t pairing, void *stream);
/* Queries of latent attention in the pool's coordinates: q_out[n, h] = [qa[h, n, :R] | rotate(q[n, h, D : D + rd], pos[n])] with qa
 * [H, N, R] the unrotated query parts already multiplied by the key up-projection, q [N, H, D + rd] with rows q_ld elements apart (a
 * column range of a wider product). */
JL_API int jl_latent_q_pack(const void *qa, const void *q, int64_t q_ld, int dtype, int64_t N, int32_t H, int32_t D, int32_t R, int32_t rd,
                            int32_t rot_dims, const int32_t *pos, const float *cos_t, const float *sin_t, int64_t table_len, void *q_out,
                            int32_t pairing, void *stream);
/* out[n, h*Dv + d] = ov[h, n, d] * sigmoid(gate[n * gate_ld + h*Dv + d]) (gate null: no gate). */
JL_API int jl_heads_gate(const void *ov, const void *gate, int64_t gate_ld, int dtype, int64_t N, int32_t H, int32_t Dv, void *out,
                         void *stream);

/* Retention (linear attention with a fixed decay per head, no denominator) over the ragged batch, state carried in float:
 *   q, k rotated (rotate-half pairs on the first rot_dims dimensions, angles from the cos / sin tables [positions, rot_dims/2]),
 *   k *= D^-1/2;   S_t = decay_h S_(t-1) + k_t v_t^T;   o_t = S_t^T q_t;
 *   out_h(t) = o_t / sqrt(mean(o_t^2) + eps) * silu(gate_h(t))
 * proj [N, ld] holds q, k (H*D columns each), v and gate (H*Dv each) at the given columns.  state [slots, H, D, Dv] float: a request
 * with pos0 == 0 starts from zero (its slot's old content is ignored), otherwise from state[slot]; the final state is written
 * back.  seq [B, 4] int32 as above.
 *
 * `mode` JL_RET_SCAN is that.  Long portions are cut into chunks that run side by side in three launches: JL_RET_LOCAL_STATE (the
 * records are chunks, `state` a scratch [chunks, H, D, Dv] indexed by the record's slot: each chunk's own contribution from a zero
 * state, no output), jl_retention_join (turns the contributions into the state every chunk starts from and writes the requests'
 * final states), JL_RET_FROM_SLOT (chunks again: outputs from the scratch's start states, nothing stored). */
#define JL_RET_SCAN 0
#define JL_RET_LOCAL_STATE 1
#define JL_RET_FROM_SLOT 2
JL_API int jl_retention(const void *proj, int dtype, int64_t ld, int32_t q_col, int32_t k_col, int32_t v_col, int32_t g_col,
                        const int32_t *seq, int32_t B, int32_t H, int32_t D, int32_t Dv, int32_t rot_dims, const float *cos_t,
                        const float *sin_t, int64_t table_len, const float *decay, float eps, float *state, void *out,
                        int32_t mode, void *stream);
/* req [B, 4] int32 = {first chunk, chunks, pos0, slot}; chunk_len [chunks] int32; scratch [chunks, H, D, Dv] float as above. */
JL_API int jl_retention_join(const int32_t *req, int32_t B, const int32_t *chunk_len, int32_t H, int32_t D, int32_t Dv,
                             const float *decay, float *state, float *scratch, void *stream);

/* Gated delta rule over the ragged batch, state carried in float.  Per head h (key head c = h / (H / G)) and token t:
 *   q, k = unit vectors (x / sqrt(sum x^2 + unit_eps)) of the head's D query / key values, q also times q_scale;
 *   beta = sigmoid(b_h(t));   g = exp(-exp(A_log[h]) * softplus(a_h(t) + dt_bias[h]));
 *   S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q            (S [D, Dv]; the read-out sees the token's own write)
 *   out_h(t) = o / sqrt(mean(o^2) + eps) * norm_w * silu(gate_h(t))             (norm_w float [Dv], shared by the heads)
 * qkv float [N, qkv_ld] holds q, k (G*D columns each) and v (H*Dv) after their convolution and activation; proj [N, ld] of `dtype` holds
 * a, b (H columns each) and the gate (H*Dv).  state [slots, H, D, Dv] float: a request with pos0 == 0 starts from zero (its slot's old
 * content is ignored); the final state is written back.  out [N, H*Dv] of `dtype`, N the batch's rows.  D <= 256, Dv <= 1024.
 * `raw` null: one workgroup per (request, head) that also normalises and gates (single tokens, short portions).  `raw` = N * H * Dv floats
 * of scratch: the form for long portions — the state's columns shared out over single-wavefront workgroups whose unnormalised outputs go
 * to `raw`, and a second launch for norm and gate. */
JL_API int jl_delta_rule(const void *qkv, int qkv_dtype, int64_t qkv_ld, int32_t q_col, int32_t k_col, int32_t v_col, const void *proj, int dtype,
                         int64_t ld, int32_t a_col, int32_t b_col, int32_t g_col, const float *A_log, const float *dt_bias, const float *norm_w,
                         const int32_t *seq, int32_t B, int64_t N, int32_t H, int32_t G, int32_t D, int32_t Dv, float unit_eps, float q_scale, float eps,
                         float *state, float *raw, void *out, void *stream);

/* Router of a mixture of experts over float logits [N, E]; ids [N, top] int32, weights [N, top] float.
 *   JL_ROUTE_SIGMOID:        s = sigmoid(logits); the `top` experts with the largest s + correction are chosen (ties: lowest
 *                            index); weights = s * scale (not renormalised).
 *   JL_ROUTE_SOFTMAX_RENORM: s = softmax(logits) over all experts; the `top` largest are chosen (ties: lowest index); weights =
 *                            s / (sum of the chosen s + renorm_eps) * scale.  `correction` is not read.
 *   JL_ROUTE_TOP_SOFTMAX:    the `top` largest logits are chosen (ties: lowest index); weights = softmax over the chosen logits
 *                            only, times scale.  `correction` is not read. */
#define JL_ROUTE_SIGMOID 0
#define JL_ROUTE_SOFTMAX_RENORM 1
#define JL_ROUTE_TOP_SOFTMAX 2
JL_API int jl_moe_route(const float *logits, const float *correction, int64_t N, int32_t E, int32_t top, float scale, int32_t *ids,
                        float *weights, int32_t kind, float renorm_eps, void *stream);

/* Rows (token, choice) grouped by expert.  perm [N*top]: sorted row -> flat index n*top + s; offsets [E+1]; tile_expert /
 * tile_row0 [max_tiles] (max_tiles >= N*top/tile_rows + E): row tiles of at most tile_rows rows of one expert, unused entries -1. */
JL_API int jl_moe_group(const int32_t *ids, int64_t N, int32_t top, int32_t E, int32_t tile_rows, int32_t *perm, int32_t *offsets,
                        int32_t *tile_expert, int32_t *tile_row0, int32_t max_tiles, void *stream);
JL_API int jl_moe_tile_rows(void);

/* Grouped product over the sorted rows: C[r, :] = X[in(r), :] . W[e(r)]^T with W [E, n_out, K].
 *   mode 0 (up):   in(r) = perm[r] / top;  out[r, :] = relu(C)^2, stored in `dtype` ([N*top, n_out], sorted order)
 *   mode 1 (down): in(r) = r;              out[perm[r], :] = C * weights[perm[r]], stored as float ([N*top, n_out])
 *   mode JL_MOE_UP_PLAIN: as mode 0 without the activation (out[r, :] = C): a gated unit stacks its gate and linear branch in W and
 *                  applies jl_gated_act to the result */
#define JL_MOE_UP_PLAIN 2
JL_API int jl_moe_gemm(const void *X, const void *Wt, int dtype, int32_t mode, int32_t K, int32_t n_out, int32_t top,
                       const int32_t *perm, const int32_t *offsets, const int32_t *tile_expert, const int32_t *tile_row0,
                       int32_t max_tiles, const float *weights, void *out, void *stream);

/* The up product of gated experts with the unit applied in its epilogue: W [E, 2*ff, K] stacks every expert's gate rows on its
 * linear rows; out[r, c] = unit(X[in(r)] . W[e(r), c], X[in(r)] . W[e(r), ff + c]) with in(r) = perm[r] / top, stored in `dtype`
 * ([N*top, ff], sorted order); kind / limit / alpha / shift as for jl_gated_act. */
JL_API int jl_moe_gemm_gated(const void *X, const void *Wt, int dtype, int32_t K, int32_t ff, int32_t top, const int32_t *perm,
                             const int32_t *offsets, const int32_t *tile_expert, const int32_t *tile_row0, int32_t max_tiles, int32_t kind,
                             float limit, float alpha, float shift, void *out, void *stream);

#ifdef __cplusplus
}
#endif
#endif
